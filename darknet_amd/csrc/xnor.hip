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
#include <float.h>
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
    /* sign bits of this layer's output for the xnor layer that reads it (NULL: none), in that layer's
     * xbits layout [batch][(n+31)/32][pixels]; and, for the kernel that also pools, the 2x2/2 maximum */
    unsigned *next_bits;
    float *pool_out;
    int ph, pw, lean; /* pooled size; lean: `out` is not written */
    long ptotal;      /* batch * ph * pw */
};

/* The tail of an output: normalize, scale, bias, activation, each step rounded to float as the
 * reference's separate passes round it (src/batchnorm_layer.c:151-154, src/activations.h:31-39).  A
 * multiplication by a double constant (the reciprocal of the batch-norm denominator, leaky's .1) is
 * fmaf(x, hi, x*lo) with the constant as an unevaluated sum of two floats: the float nearest the
 * double product except within ~2^-48 of a rounding boundary, without the three double-precision
 * instructions that made this tail the larger part of the early layers (nine words of bit work
 * per output at 16 input channels). */
struct xn_f2 {
    float hi, lo;
};
__device__ __forceinline__ xn_f2 xn_split(double c)
{
    xn_f2 r;
    r.hi = (float)c;
    r.lo = (float)(c - (double)r.hi);
    return r;
}
struct xn_row {
    xn_f2 inv;
    float mean, scale, bias, wmean;
};
/* ACT: 0 = leaky, 1 = linear, 2 = relu (branch-free forms), 3 = any other (the general switch) */
template <int ACT>
__device__ __forceinline__ float xn_tail(float acc, const xn_row &r, int act)
{
    const float d = __fsub_rn(acc, r.mean);
    float x = fmaf(d, r.inv.hi, __fmul_rn(d, r.inv.lo));
    x = __fadd_rn(__fmul_rn(x, r.scale), r.bias);
    if (ACT == 0) {
        const xn_f2 s = xn_split(.1);
        return x > 0 ? x : fmaf(x, s.hi, __fmul_rn(x, s.lo));
    }
    if (ACT == 1) return x;
    if (ACT == 2) return x * (float)(x > 0);
    return dn_activate(x, act);
}

/* 3x3 kernels with a padding of at most one pixel: the taps of an output that fall outside the
 * image are a row (the first or the last), a column, or both - nine classes, 3*cy + cx with cy, cx
 * in {0 none, 1 first, 2 last}.  A tap outside contributes a zero word, which counts popcount(w) as
 * mismatches; corr[j][class] is that miscount for filter j, taken from the per-tap popcounts once
 * per workgroup, so that an output pays one LDS read and one subtraction for it. */
__device__ __forceinline__ void xn_fill_corr(int *corr, const int *__restrict__ wpop, int f0, int n)
{
    if (threadIdx.x < XN_FPB * 9) {
        const int j = threadIdx.x / 9, cls = threadIdx.x - 9 * j, cy = cls / 3, cx = cls - 3 * cy;
        int s = 0;
        if (f0 + j < n)
#pragma unroll
            for (int t = 0; t < 9; ++t) {
                const int ky = t / 3, kx = t % 3;
                const bool out = (cy == 1 && ky == 0) || (cy == 2 && ky == 2) || (cx == 1 && kx == 0) || (cx == 2 && kx == 2);
                if (out) s += wpop[(f0 + j) * 9 + t];
            }
        corr[threadIdx.x] = s;
    }
}
/* class of an output whose window starts at i0 in an axis of length len (pad <= 1, len >= 2) */
__device__ __forceinline__ int xn_axis_class(int i0, int len) { return i0 < 0 ? 1 : (i0 + 2 >= len ? 2 : 0); }

/* The 16 sign bits a workgroup made for pixel p of image b, into the xbits of the layer that reads
 * this one: word (b, f0/32, p), lower or upper half by f0.  Two workgroups fill the halves of a
 * word; where the upper half has no filters (the last 16-filter block of an odd count) the lower
 * one's lane writes the whole word, so the buffer needs no clearing. */
__device__ __forceinline__ void xn_store_bits(unsigned *next_bits, unsigned bits, int f0, int n, int b, int P, int p)
{
    const int cwn = (n + 31) >> 5;
    unsigned *word = next_bits + ((long)b * cwn + (f0 >> 5)) * P + p;
    if ((f0 & 16) == 0 && f0 + 16 >= n)
        *word = bits;
    else
        ((unsigned short *)word)[(f0 >> 4) & 1] = (unsigned short)bits;
}

/* 3x3 / stride 1 / pad 1 convolution followed by the 2x2 stride-2 maximum of the maxpool layer
 * behind it (src/maxpool_layer.c:79-114 with size 2, stride 2, padding 1: windows start at even
 * pixels and never leave an image of even size), in one pass.  A lane owns one pooled pixel, i.e. a
 * 2x2 quad of convolution outputs, and 16 filters: per 32-channel slice it loads the 4x4 words the
 * quad's taps touch once (16 loads for 36 tap reads) and index arithmetic, filter constants and
 * stores are shared by four outputs.  It writes the convolution's map (two 8-byte stores per
 * filter; skipped when `lean`), the pooled map, and, when asked, the sign bits of the pooled map
 * for the xnor layer behind the pool.  The pooled value is the window-order maximum of the four
 * finished outputs, as the pooling layer computes it.  When the map is not written and the tail is
 * monotone in the integer dot product (leaky, linear, relu: then it rises with the dot product for a
 * scale >= 0 and falls for a negative one, rounding included), the tail runs once, on the largest
 * (smallest) of the four dot products: the same value, a quarter of the arithmetic. */
template <int ACT>
__global__ __launch_bounds__(XN_BLOCK) void xnor_conv_pool_kernel(const unsigned *__restrict__ xbits,
                                                                  const unsigned *__restrict__ wbits,
                                                                  const int *__restrict__ wpop, xnor_args a)
{
    const int f0 = blockIdx.y * XN_FPB;
    __shared__ xn_row rows[XN_FPB];
    if (threadIdx.x < XN_FPB && f0 + (int)threadIdx.x < a.n) {
        const int f = f0 + threadIdx.x;
        xn_row r;
        r.wmean = a.wmean[f];
        r.bias = a.biases[f];
        r.mean = a.bn ? a.mean[f] : 0.f;
        r.scale = a.bn ? a.scales[f] : 1.f;
        r.inv = xn_split(a.bn ? 1.0 / (sqrt((double)a.var[f]) + (double).000001f) : 1.0);
        rows[threadIdx.x] = r;
    }
    __shared__ int corr[XN_FPB * 9];
    xn_fill_corr(corr, wpop, f0, a.n);
    __syncthreads();
    const unsigned col = blockIdx.x * (unsigned)XN_BLOCK + threadIdx.x; /* the host keeps ptotal below 2^31 */
    const bool col_ok = col < (unsigned)a.ptotal;
    const unsigned cc = col_ok ? col : 0u;
    const unsigned PP = (unsigned)(a.ph * a.pw);
    const int b = (int)(cc / PP);
    const int pp = (int)(cc - (unsigned)b * PP);
    const int py = pp / a.pw, px = pp - py * a.pw;
    const int iy0 = 2 * py - 1, ix0 = 2 * px - 1;
    const int plane = a.h * a.w;
    const unsigned *xb = xbits + (long)b * a.cw * plane;
    /* the 4x4 window: bit 4*r+q of `valid` says that word lies inside the image */
    unsigned valid = 0;
    int off[16];
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int iy = iy0 + r, ix = ix0 + q;
            const bool in = iy >= 0 && iy < a.h && ix >= 0 && ix < a.w;
            if (in) valid |= 1u << (4 * r + q);
            off[4 * r + q] = in ? iy * a.w + ix : 0;
        }
    int mism[4][XN_FPB];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < XN_FPB; ++j) mism[i][j] = 0;
    for (int wd = 0; wd < a.cw; ++wd) {
        const unsigned *xw = xb + (long)wd * plane;
        unsigned x[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) x[i] = xw[off[i]];
#pragma unroll
        for (int i = 0; i < 16; ++i) x[i] = ((valid >> i) & 1u) ? x[i] : 0u;
#pragma unroll
        for (int t = 0; t < 9; ++t) {
            const unsigned *wrow = wbits + ((long)t * a.cw + wd) * a.npad + f0; /* wave-uniform */
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const unsigned xv = x[((i >> 1) + t / 3) * 4 + (i & 1) + t % 3];
#pragma unroll
                for (int j = 0; j < XN_FPB; ++j) mism[i][j] += __popc(xv ^ wrow[j]);
            }
        }
    }
    if (!col_ok) return;
    /* border class of each output of the quad (pad 1, stride 1: output y's window starts at y - 1) */
    int cls[4], inside_c[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int cy = xn_axis_class(2 * py + (i >> 1) - 1, a.h), cx = xn_axis_class(2 * px + (i & 1) - 1, a.w);
        cls[i] = 3 * cy + cx;
        inside_c[i] = (cy ? 2 : 3) * (cx ? 2 : 3) * a.c;
    }
    const int P = a.oh * a.ow;
    const long PPl = (long)a.ph * a.pw;
    unsigned bits = 0;
#pragma unroll
    for (int j = 0; j < XN_FPB; ++j) {
        const int f = f0 + j;
        if (f >= a.n) continue;
        int dot[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) dot[i] = inside_c[i] - 2 * (mism[i][j] - corr[j * 9 + cls[i]]);
        const xn_row row = rows[j];
        float pooled;
        if (a.lean && ACT != 3) {
            const int hi = max(max(dot[0], dot[1]), max(dot[2], dot[3]));
            const int lo = min(min(dot[0], dot[1]), min(dot[2], dot[3]));
            const float v = xn_tail<ACT>(__fmul_rn(row.wmean, (float)(row.scale >= 0.f ? hi : lo)), row, a.act);
            pooled = v > -FLT_MAX ? v : -FLT_MAX;
        } else {
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = xn_tail<ACT>(__fmul_rn(row.wmean, (float)dot[i]), row, a.act);
            pooled = -FLT_MAX;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (v[i] > pooled) pooled = v[i];
            if (!a.lean) {
                float *o = a.out + ((long)b * a.n + f) * P + (long)(2 * py) * a.ow + 2 * px;
                *(float2 *)o = make_float2(v[0], v[1]);
                *(float2 *)(o + a.ow) = make_float2(v[2], v[3]);
            }
        }
        a.pool_out[((long)b * a.n + f) * PPl + pp] = pooled;
        if (pooled > 0) bits |= 1u << j;
    }
    if (a.next_bits) xn_store_bits(a.next_bits, bits, f0, a.n, b, (int)PPl, pp);
}

/* SIZE = 3 or 1: the taps are unrolled and, per 32-channel slice, the words of all taps are
 * requested before the first is used (one trip to memory per slice instead of one per tap; with
 * a loop over taps of a size known only at run time a wave stood through nine dependent trips).
 * SIZE = 0: any kernel size, taps in a run-time loop. */
template <int ACT, int SIZE, bool BITS>
__global__ __launch_bounds__(XN_BLOCK) void xnor_conv_kernel(const unsigned *__restrict__ xbits,
                                                             const unsigned *__restrict__ wbits,
                                                             const int *__restrict__ wpop, xnor_args a)
{
    const int ss = a.size * a.size;
    const int f0 = blockIdx.y * XN_FPB;
    const int P = a.oh * a.ow;
    /* the batch-norm constants of the workgroup's filters (a double square root and division
     * each) are the same for every pixel: computed once, by one lane per filter */
    __shared__ xn_row rows[XN_FPB];
    if (threadIdx.x < XN_FPB && f0 + (int)threadIdx.x < a.n) {
        const int f = f0 + threadIdx.x;
        xn_row r;
        r.wmean = a.wmean[f];
        r.bias = a.biases[f];
        r.mean = a.bn ? a.mean[f] : 0.f;
        r.scale = a.bn ? a.scales[f] : 1.f;
        r.inv = xn_split(a.bn ? 1.0 / (sqrt((double)a.var[f]) + (double).000001f) : 1.0);
        rows[threadIdx.x] = r;
    }
    __shared__ int corr[XN_FPB * 9];
    if (SIZE == 3) xn_fill_corr(corr, wpop, f0, a.n);
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
    if (SIZE > 0) {
        constexpr int SS = SIZE > 0 ? SIZE * SIZE : 1;
        int off[SS];
#pragma unroll
        for (int t = 0; t < SS; ++t) {
            const int iy = iy0 + t / SIZE, ix = ix0 + t % SIZE;
            const bool inside = iy >= 0 && iy < a.h && ix >= 0 && ix < a.w;
            if (!inside) outside |= 1u << t;
            off[t] = inside ? iy * a.w + ix : 0;
        }
        for (int wd = 0; wd < a.cw; ++wd) {
            const unsigned *xw = xb + wd * plane;
            unsigned x[SS];
#pragma unroll
            for (int t = 0; t < SS; ++t) x[t] = xw[off[t]];
#pragma unroll
            for (int t = 0; t < SS; ++t) {
                const unsigned xv = ((outside >> t) & 1u) ? 0u : x[t];
                const unsigned *wrow = wbits + ((long)t * a.cw + wd) * a.npad + f0; /* wave-uniform */
#pragma unroll
                for (int j = 0; j < XN_FPB; ++j) mism[j] += __popc(xv ^ wrow[j]);
            }
        }
    } else {
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
    }
    if (!col_ok) return;
    const int taps_inside = ss - __popc(outside);
    const int cls = SIZE == 3 ? 3 * xn_axis_class(iy0, a.h) + xn_axis_class(ix0, a.w) : 0;
    unsigned bits = 0;
#pragma unroll
    for (int j = 0; j < XN_FPB; ++j) {
        const int f = f0 + j;
        if (f >= a.n) continue;
        int m = mism[j];
        if (SIZE == 3)
            m -= corr[j * 9 + cls];
        else if (SIZE == 0)
            for (unsigned o = outside; o; o &= o - 1) m -= wpop[f * ss + (__ffs(o) - 1)];
        const int dot = taps_inside * a.c - 2 * m;
        const float acc = __fmul_rn(rows[j].wmean, (float)dot);
        const float v = xn_tail<ACT>(acc, rows[j], a.act);
        a.out[((long)b * a.n + f) * P + p] = v;
        if (BITS && v > 0) bits |= 1u << j;
    }
    if (BITS) xn_store_bits(a.next_bits, bits, f0, a.n, b, P, p);
}

template <int SIZE, bool BITS>
static void xnor_launch(dim3 grid, const unsigned *xbits, const unsigned *wbits, const int *wpop, const xnor_args &a,
                        int activation)
{
    void (*kernel)(const unsigned *, const unsigned *, const int *, xnor_args) =
        activation == DN_LEAKY ? xnor_conv_kernel<0, SIZE, BITS> : activation == DN_LINEAR ? xnor_conv_kernel<1, SIZE, BITS>
        : activation == DN_RELU ? xnor_conv_kernel<2, SIZE, BITS> : xnor_conv_kernel<3, SIZE, BITS>;
    hipLaunchKernelGGL(kernel, grid, dim3(XN_BLOCK), 0, dn_stream(), xbits, wbits, wpop, a);
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

extern "C" void forward_convolutional_xnor_fused_gpu(const float *input, const unsigned *wbits, const float *wmean,
                                                     unsigned *xbits, int xbits_ready, const float *biases,
                                                     const float *scales, const float *rolling_mean,
                                                     const float *rolling_variance, float *output,
                                                     float *pool_output, unsigned *next_xbits, int batch, int c,
                                                     int h, int w, int n, int size, int stride, int pad,
                                                     int batch_normalize, int activation)
{
    if (batch <= 0 || c <= 0 || h <= 0 || w <= 0 || n <= 0 || size <= 0 || stride <= 0 || pad < 0)
        dn_fatal("forward_convolutional_xnor_gpu: bad geometry");
    if ((!input && !xbits_ready) || !wbits || !wmean || !xbits || !biases || (!output && !pool_output))
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
    if ((long)batch * a.cw * h * w >= (1L << 31) || (long)h * w * a.cw >= (1L << 31))
        dn_fatal("forward_convolutional_xnor_gpu: input too large");
    /* the input is binarised on every forward (src/convolutional_layer.c:454) unless the layer
     * that produced it wrote the bits already */
    if (!xbits_ready) xnor_pack_input_gpu(input, xbits, batch, c, h, w);
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
    a.next_bits = next_xbits;
    a.pool_out = pool_output;
    a.ph = a.oh / 2;
    a.pw = a.ow / 2;
    a.ptotal = (long)batch * a.ph * a.pw;
    a.lean = output ? 0 : 1;
    const int fblocks = (n + XN_FPB - 1) / XN_FPB;
    const int *wpop = (const int *)(wbits + (long)size * size * a.cw * a.npad);
    if (pool_output) {
        if (size != 3 || stride != 1 || pad != 1 || (a.oh & 1) || (a.ow & 1) || h < 2 || w < 2)
            dn_fatal("forward_convolutional_xnor_fused_gpu: the pooled form serves 3x3 / stride 1 / pad 1 layers of even size");
        if (a.ptotal >= (1L << 31) - XN_BLOCK) dn_fatal("forward_convolutional_xnor_fused_gpu: output too large");
        const long cblocks = (a.ptotal + XN_BLOCK - 1) / XN_BLOCK;
        if (fblocks > 65535) dn_fatal("forward_convolutional_xnor_gpu: grid too large");
        dim3 grid((unsigned)cblocks, fblocks, 1);
        void (*kernel)(const unsigned *, const unsigned *, const int *, xnor_args) =
            activation == DN_LEAKY ? xnor_conv_pool_kernel<0> : activation == DN_LINEAR ? xnor_conv_pool_kernel<1>
            : activation == DN_RELU ? xnor_conv_pool_kernel<2> : xnor_conv_pool_kernel<3>;
        hipLaunchKernelGGL(kernel, grid, dim3(XN_BLOCK), 0, dn_stream(), (const unsigned *)xbits, wbits, wpop, a);
        dn_check_launch("forward_convolutional_xnor_fused_gpu");
        return;
    }
    const long cblocks = (a.ntotal + XN_BLOCK - 1) / XN_BLOCK;
    if (fblocks > 65535 || cblocks >= (1L << 31)) dn_fatal("forward_convolutional_xnor_gpu: grid too large");
    dim3 grid((unsigned)cblocks, fblocks, 1);
    const unsigned *xb = (const unsigned *)xbits;
    const bool three = size == 3 && pad <= 1 && h >= 2 && w >= 2; /* the nine border classes of xn_fill_corr */
    if (next_xbits) {
        if (three) xnor_launch<3, true>(grid, xb, wbits, wpop, a, activation);
        else if (size == 1) xnor_launch<1, true>(grid, xb, wbits, wpop, a, activation);
        else xnor_launch<0, true>(grid, xb, wbits, wpop, a, activation);
    } else {
        if (three) xnor_launch<3, false>(grid, xb, wbits, wpop, a, activation);
        else if (size == 1) xnor_launch<1, false>(grid, xb, wbits, wpop, a, activation);
        else xnor_launch<0, false>(grid, xb, wbits, wpop, a, activation);
    }
    dn_check_launch("forward_convolutional_xnor_gpu");
}

extern "C" void forward_convolutional_xnor_packed_gpu(const float *input, const unsigned *wbits,
                                                      const float *wmean, unsigned *xbits, const float *biases,
                                                      const float *scales, const float *rolling_mean,
                                                      const float *rolling_variance, float *output, int batch,
                                                      int c, int h, int w, int n, int size, int stride, int pad,
                                                      int batch_normalize, int activation)
{
    if (!input || !output) dn_fatal("forward_convolutional_xnor_gpu: null pointer");
    forward_convolutional_xnor_fused_gpu(input, wbits, wmean, xbits, 0, biases, scales, rolling_mean, rolling_variance,
                                         output, 0, 0, batch, c, h, w, n, size, stride, pad, batch_normalize,
                                         activation);
}
