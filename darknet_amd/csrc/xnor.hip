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
 *   wbits [size*size][Cw][Npad]  filters innermost (Npad = n rounded up to 16, padding 0): the 16
 *                                 filters a workgroup works on are 64 contiguous bytes per
 *                                 (tap, slice), fetched with ONE scalar load and used straight
 *                                 from scalar registers - the filter operand costs no vector
 *                                 register, no LDS and no vector instruction
 *   wpop  [n][size*size]         popcount of a filter's bits per tap, stored behind wbits
 *
 * Kernel: a lane owns one output pixel (columns run over batch*out_h*out_w, so every wavefront is
 * full whatever the image size) and 16 filters; per (tap, slice) it loads one word of xbits and
 * does 16 x (v_xor with a scalar operand, v_bcnt with accumulate).  Taps outside the image load
 * a zero word instead of branching; what the zero word miscounts, popcount(w), is taken back at
 * the end from wpop.
 */
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_math.h"
#include "hip.h"

#define XN_BLOCK 256
#define XN_FPB 16 /* filters per workgroup */

static inline hipStream_t dn_stream() { return (hipStream_t)hip_get_stream(); }

static inline int xnor_npad(int n) { return (n + XN_FPB - 1) / XN_FPB * XN_FPB; }

/* words of wbits followed by wpop */
extern "C" size_t xnor_weight_words(int n, int c, int size)
{
    return (size_t)xnor_npad(n) * size * size * ((c + 31) / 32) + (size_t)n * size * size;
}

extern "C" size_t xnor_input_words(int batch, int c, int h, int w)
{
    return (size_t)batch * ((c + 31) / 32) * h * w;
}

/* One workgroup of two wavefronts per filter.  Lane 0 of the first takes the |w| sum, which must
 * run in the reference's order to round alike (a chain of K dependent additions); the second
 * packs the sign bits, one (tap, slice) word per lane and trip, and the per-tap popcounts. */
__global__ __launch_bounds__(128) void xnor_pack_weights_kernel(const float *weights, unsigned *wbits, int *wpop,
                                                                float *wmean, int n, int npad, int c, int size)
{
    const int f = blockIdx.x;
    const int ss = size * size;
    const int K = c * ss;
    const int cw = (c + 31) / 32;
    const float *w = weights + (long)f * K;
    if (threadIdx.x == 0) {
        float mean = 0;
        for (int i = 0; i < K; ++i) mean = (float)((double)mean + fabs((double)w[i]));
        wmean[f] = mean / K;
    } else if (threadIdx.x >= 64) {
        const int lane = threadIdx.x - 64;
        for (int t = 0; t < ss; ++t) {
            int pop = 0;
            for (int wd = lane; wd < cw; wd += 64) {
                unsigned bits = 0;
                for (int j = 0; j < 32; ++j) {
                    const int ch = wd * 32 + j;
                    if (ch < c && w[(long)ch * ss + t] > 0) bits |= 1u << j;
                }
                wbits[((long)t * cw + wd) * npad + f] = bits;
                pop += __popc(bits);
            }
            for (int o = 32; o > 0; o >>= 1) pop += __shfl_xor(pop, o);
            if (lane == 0) wpop[f * ss + t] = pop;
        }
    }
}

__global__ void xnor_clear_pad_kernel(unsigned *wbits, int n, int npad, long rows)
{
    const int padn = npad - n;
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < rows * padn; i += (long)gridDim.x * blockDim.x)
        wbits[(i / padn) * npad + n + (i % padn)] = 0u;
}

extern "C" void xnor_pack_weights_gpu(const float *weights, unsigned *wbits, float *wmean, int n, int c,
                                      int size)
{
    if (hip_parse_only()) return;
    const int npad = xnor_npad(n);
    const long rows = (long)size * size * ((c + 31) / 32);
    int *wpop = (int *)(wbits + rows * npad);
    if (npad != n)
        hipLaunchKernelGGL(xnor_clear_pad_kernel, dim3(64), dim3(256), 0, dn_stream(), wbits, n, npad, rows);
    hipLaunchKernelGGL(xnor_pack_weights_kernel, dim3(n), dim3(128), 0, dn_stream(), weights, wbits, wpop, wmean,
                       n, npad, c, size);
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
    const float *wmean;
    const float *biases, *scales, *mean, *var;
    float *out;
    int c, h, w, n, npad, size, stride, pad, oh, ow, cw, bn, act;
    long ntotal; /* batch * oh * ow */
};

__global__ __launch_bounds__(XN_BLOCK) void xnor_conv_kernel(const unsigned *__restrict__ xbits,
                                                             const unsigned *__restrict__ wbits,
                                                             const int *__restrict__ wpop, xnor_args a)
{
    const int ss = a.size * a.size;
    const int f0 = blockIdx.y * XN_FPB;
    const int P = a.oh * a.ow;
    /* the batch-norm constants of the workgroup's filters (a double square root and division
     * each) are the same for every pixel: computed once, by one lane per filter */
    __shared__ dn_bn_row rows[XN_FPB];
    __shared__ float wmeans[XN_FPB];
    if (threadIdx.x < XN_FPB && f0 + (int)threadIdx.x < a.n) {
        const int f = f0 + threadIdx.x;
        rows[threadIdx.x] = dn_bn_make(a.bn, a.biases[f], a.bn ? a.scales[f] : 1.f, a.bn ? a.mean[f] : 0.f,
                                       a.bn ? a.var[f] : 1.f);
        wmeans[threadIdx.x] = a.wmean[f];
    }
    __syncthreads();
    const long col = blockIdx.x * (long)XN_BLOCK + threadIdx.x;
    const bool col_ok = col < a.ntotal;
    const long cc = col_ok ? col : 0;
    const int b = (int)(cc / P);
    const int p = (int)(cc - (long)b * P);
    const int oy = p / a.ow, ox = p - oy * a.ow;
    const int iy0 = oy * a.stride - a.pad, ix0 = ox * a.stride - a.pad;
    const long plane = (long)a.h * a.w;
    const unsigned *xb = xbits + (long)b * a.cw * plane;
    int mism[XN_FPB];
#pragma unroll
    for (int j = 0; j < XN_FPB; ++j) mism[j] = 0;
    unsigned outside = 0; /* bit t: tap t lies outside the image for this lane */
    int t = 0;
    for (int ky = 0; ky < a.size; ++ky) {
        for (int kx = 0; kx < a.size; ++kx, ++t) {
            const int iy = iy0 + ky, ix = ix0 + kx;
            const bool inside = iy >= 0 && iy < a.h && ix >= 0 && ix < a.w;
            if (!inside) outside |= 1u << t;
            const unsigned *xp = xb + (inside ? (long)iy * a.w + ix : 0);
            const unsigned *wrow = wbits + (long)t * a.cw * a.npad + f0; /* wave-uniform */
#pragma unroll 4
            for (int wd = 0; wd < a.cw; ++wd) {
                const unsigned xv = xp[wd * plane];
                const unsigned x = inside ? xv : 0u;
#pragma unroll
                for (int j = 0; j < XN_FPB; ++j) mism[j] += __popc(x ^ wrow[(long)wd * a.npad + j]);
            }
        }
    }
    if (!col_ok) return;
    const int taps_inside = ss - __popc(outside);
#pragma unroll
    for (int j = 0; j < XN_FPB; ++j) {
        const int f = f0 + j;
        if (f >= a.n) break;
        int m = mism[j];
        for (unsigned o = outside; o; o &= o - 1) m -= wpop[f * ss + (__ffs(o) - 1)];
        const int dot = taps_inside * a.c - 2 * m;
        const float acc = __fmul_rn(wmeans[j], (float)dot);
        a.out[((long)b * a.n + f) * P + p] = dn_activate(dn_bn_apply(acc, rows[j], a.bn), a.act);
    }
}

extern "C" void forward_convolutional_xnor_packed_gpu(const float *input, const unsigned *wbits,
                                                      const float *wmean, unsigned *xbits, const float *biases,
                                                      const float *scales, const float *rolling_mean,
                                                      const float *rolling_variance, float *output, int batch,
                                                      int c, int h, int w, int n, int size, int stride, int pad,
                                                      int batch_normalize, int activation);

extern "C" void forward_convolutional_xnor_gpu(const float *input, const float *weights, unsigned *wbits,
                                               float *wmean, unsigned *xbits, const float *biases,
                                               const float *scales, const float *rolling_mean,
                                               const float *rolling_variance, float *output, int batch,
                                               int c, int h, int w, int n, int size, int stride, int pad,
                                               int batch_normalize, int activation)
{
    if (!weights || !wbits || !wmean) dn_fatal("forward_convolutional_xnor_gpu: null pointer");
    if (n <= 0 || c <= 0 || size <= 0) dn_fatal("forward_convolutional_xnor_gpu: bad geometry");
    /* the reference re-binarises the weights on every forward (src/convolutional_layer.c:451-453) */
    xnor_pack_weights_gpu(weights, wbits, wmean, n, c, size);
    forward_convolutional_xnor_packed_gpu(input, wbits, wmean, xbits, biases, scales, rolling_mean,
                                          rolling_variance, output, batch, c, h, w, n, size, stride, pad,
                                          batch_normalize, activation);
}

extern "C" void forward_convolutional_xnor_packed_gpu(const float *input, const unsigned *wbits,
                                                      const float *wmean, unsigned *xbits, const float *biases,
                                                      const float *scales, const float *rolling_mean,
                                                      const float *rolling_variance, float *output, int batch,
                                                      int c, int h, int w, int n, int size, int stride, int pad,
                                                      int batch_normalize, int activation)
{
    if (batch <= 0 || c <= 0 || h <= 0 || w <= 0 || n <= 0 || size <= 0 || stride <= 0 || pad < 0)
        dn_fatal("forward_convolutional_xnor_gpu: bad geometry");
    if (!input || !wbits || !wmean || !xbits || !biases || !output)
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
    if (size * size > 32) dn_fatal("forward_convolutional_xnor_gpu: kernels beyond 5x5 are not supported");
    /* the input is binarised on every forward (src/convolutional_layer.c:454) */
    xnor_pack_input_gpu(input, xbits, batch, c, h, w);
    a.wmean = wmean;
    a.npad = xnor_npad(n);
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
    a.ntotal = (long)batch * a.oh * a.ow;
    const int fblocks = (n + XN_FPB - 1) / XN_FPB;
    const long cblocks = (a.ntotal + XN_BLOCK - 1) / XN_BLOCK;
    if (fblocks > 65535 || cblocks >= (1L << 31)) dn_fatal("forward_convolutional_xnor_gpu: grid too large");
    const int *wpop = (const int *)(wbits + (long)size * size * a.cw * a.npad);
    dim3 grid((unsigned)cblocks, fblocks, 1);
    hipLaunchKernelGGL(xnor_conv_kernel, grid, dim3(XN_BLOCK), 0, dn_stream(), (const unsigned *)xbits,
                       (const unsigned *)wbits, wpop, a);
    dn_check_launch("forward_convolutional_xnor_gpu");
}
