/*
 * conv_group.hip - grouped 3x3 convolutions with few channels per group: 4 or 8 in and as many out
 * (src/convolutional_layer.c:445-485 with l.groups > 1: one im2col + GEMM per group; the ResNeXt
 * blocks with 32 groups of 4 and 8 channels), pad 1, stride 1 (4 per group also stride 2).
 *
 * Such a layer is 36 or 72 multiply-adds per output: on the matrix cores, where a 32-filter tile
 * multiplies a block-diagonal weight matrix, seven eighths (three quarters) of the work is zeros, and
 * the layer is not far from memory-bound to begin with.  Here it runs on the vector ALU:
 *
 *   - a workgroup owns one image, one group and a tile of 8 x 32 output pixels; the group's input
 *     channels of the tile (with their one-pixel border, zeros outside the image) are copied to LDS
 *     once; a lane owns one output pixel and all of the group's filters;
 *   - the group's weights are read through the scalar cache (every index is uniform over the
 *     workgroup) and used straight from scalar registers as the second operand of the multiply-adds:
 *     no vector register, no LDS traffic for weights;
 *   - per (channel, tap) one LDS read feeds CG multiply-adds; with stride 2 the patch keeps even and
 *     odd columns apart, so that the 32 lanes of a row read consecutive words either way;
 *   - the sum runs over k = (channel, ky, kx) in the reference's order; batch-norm, bias and
 *     activation are the tail every convolution kernel here applies (dn_tail).
 */
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_math.h"
#include "hip.h"

#define CG_THREADS 256
#define CG_RPT 1 /* output rows per lane (2 was measured: the shared patch rows save LDS reads, but the weights of
                  * twice the multiply-adds no longer fit the scalar registers: 115 against 92 us) */
#define CG_TR (8 * CG_RPT) /* output rows of a tile */
#define CG_TC 32 /* output columns of a tile */

static inline hipStream_t dn_stream() { return (hipStream_t)hip_get_stream(); }

struct group_args {
    const float *in;      /* [B][C][H][W] */
    const float *w;       /* [N][CG][3][3] */
    const float *biases, *scales, *mean, *var;
    float *out;           /* [B][N][OH][OW] */
    int C, H, W, N, OH, OW, bn;
    int tiles_x;          /* tiles across the output */
    float slope_hi, slope_lo;
};

template <int CG, int S>
__global__ __launch_bounds__(CG_THREADS) void conv_group_kernel(group_args a)
{
    constexpr int PROWS = (CG_TR - 1) * S + 3; /* input rows a tile touches: 10 or 17 */
    constexpr int PCOLS = (CG_TC - 1) * S + 3; /* input columns: 34 or 65 */
    constexpr int HALF = (PCOLS + 1) / 2;      /* stride 2: even columns first, odd columns behind them */
    constexpr int RSL = S == 1 ? PCOLS : 2 * HALF;
    __shared__ float patch[CG * PROWS * RSL];
    __shared__ dn_tail_row rows[CG];
    const int tid = threadIdx.x;
    const int tx = blockIdx.x % a.tiles_x, ty = blockIdx.x / a.tiles_x;
    const int g = blockIdx.y, b = blockIdx.z;
    const int oy0 = ty * CG_TR, ox0 = tx * CG_TC;
    const int iy0 = oy0 * S - 1, ix0 = ox0 * S - 1;
    const float *in = a.in + ((long)b * a.C + (long)g * CG) * a.H * a.W;

    if (tid < CG) {
        const int m = g * CG + tid;
        rows[tid] = dn_tail_make(a.bn, a.biases[m], a.bn ? a.scales[m] : 1.f, a.bn ? a.mean[m] : 0.f,
                                 a.bn ? a.var[m] : 1.f);
    }
    /* the patch, element by element over the workgroup (measured against a (channel, row) per wave with a
     * column per lane, which leaves half the lanes of a 34-column row idle: 92 against 105 us on
     * 128 channels at 56 x 56, batch 64) */
    for (int e = tid; e < CG * PROWS * PCOLS; e += CG_THREADS) {
        const int ch = e / (PROWS * PCOLS), rem = e - ch * (PROWS * PCOLS);
        const int r = rem / PCOLS, pc = rem - r * PCOLS;
        const int iy = iy0 + r, ix = ix0 + pc;
        const bool inside = (unsigned)iy < (unsigned)a.H && (unsigned)ix < (unsigned)a.W;
        const float v = inside ? in[((long)ch * a.H + iy) * a.W + ix] : 0.f;
        patch[(ch * PROWS + r) * RSL + (S == 1 ? pc : (pc & 1) * HALF + (pc >> 1))] = v;
    }
    __syncthreads();

    const int r = (tid >> 5) * CG_RPT, c = tid & 31; /* this lane's first output row of the tile, and its column */
    const float *wg = a.w + (long)g * CG * CG * 9; /* the group's filters: [f][ch][ky][kx], uniform over the workgroup */
    float acc[CG_RPT][CG];
#pragma unroll
    for (int j = 0; j < CG_RPT; ++j)
#pragma unroll
        for (int f = 0; f < CG; ++f) acc[j][f] = 0.f;
#pragma unroll
    for (int ch = 0; ch < CG; ++ch) {
        /* the patch rows the lane's outputs touch, three taps each */
        constexpr int NR = (CG_RPT - 1) * S + 3;
        float x[NR][3];
#pragma unroll
        for (int pr = 0; pr < NR; ++pr)
#pragma unroll
            for (int kx = 0; kx < 3; ++kx)
                x[pr][kx] = patch[(ch * PROWS + r * S + pr) * RSL + (S == 1 ? c + kx : (kx & 1) * HALF + c + (kx >> 1))];
#pragma unroll
        for (int ky = 0; ky < 3; ++ky)
#pragma unroll
            for (int kx = 0; kx < 3; ++kx)
#pragma unroll
                for (int f = 0; f < CG; ++f) {
                    const float wv = wg[(f * CG + ch) * 9 + ky * 3 + kx];
#pragma unroll
                    for (int j = 0; j < CG_RPT; ++j) acc[j][f] = fmaf(x[j * S + ky][kx], wv, acc[j][f]);
                }
    }

    const int ox = ox0 + c;
    if (ox >= a.OW) return;
    const dn_f2 slope = {a.slope_hi, a.slope_lo};
    const long plane = (long)a.OH * a.OW;
#pragma unroll
    for (int j = 0; j < CG_RPT; ++j) {
        const int oy = oy0 + r + j;
        if (oy >= a.OH) break;
        float *out = a.out + (((long)b * a.N + (long)g * CG) * a.OH + oy) * a.OW + ox;
#pragma unroll
        for (int f = 0; f < CG; ++f) out[f * plane] = dn_tail(acc[j][f], rows[f], slope);
    }
}

/* Whether conv_group_kernel serves the layer. */
extern "C" int conv_group_serves(int batch, int c, int h, int w, int n, int groups, int size, int stride, int pad)
{
    if (groups <= 1 || size != 3 || pad != 1 || (stride != 1 && stride != 2)) return 0;
    if (c % groups || n % groups || c / groups != n / groups) return 0;
    const int cg = c / groups;
    if (cg != 4 && cg != 8) return 0;
    /* 8 per group at stride 2: the patch is four times the outputs' area and eight channels deep, and the
     * block-diagonal tiles of the matrix cores win (137 against 158 us on 256 channels at 56 x 56, batch 64) */
    if (cg == 8 && stride == 2) return 0;
    if (batch < 1 || batch > 65535 || groups > 65535 || h < 1 || w < 1) return 0;
    const int oh = (h + 2 - 3) / stride + 1, ow = (w + 2 - 3) / stride + 1;
    if (oh < 1 || ow < 1) return 0;
    if ((long)((oh + CG_TR - 1) / CG_TR) * ((ow + CG_TC - 1) / CG_TC) >= (1L << 31)) return 0;
    if ((long)h * w >= (1L << 28)) return 0; /* a group's channels of one image are indexed in 32 bits */
    return 1;
}

extern "C" const char *conv_group_kernel_name(int c, int groups, int stride)
{
    const int cg = c / groups;
    return cg == 4 ? (stride == 1 ? "conv_group_kernel<4,1>" : "conv_group_kernel<4,2>") : "conv_group_kernel<8,1>";
}

/* The launch.  slope: the activation as y > 0 ? y : slope*y (leaky .1, linear 1, relu 0). */
extern "C" void conv_group_forward(const float *input, const float *weights, const float *biases, const float *scales,
                                   const float *rolling_mean, const float *rolling_variance, float *output, int batch,
                                   int c, int h, int w, int n, int groups, int stride, int batch_normalize, double slope)
{
    if (!conv_group_serves(batch, c, h, w, n, groups, 3, stride, 1)) dn_fatal("conv_group_forward: geometry not served");
    group_args a;
    a.in = input;
    a.w = weights;
    a.biases = biases;
    a.scales = scales;
    a.mean = rolling_mean;
    a.var = rolling_variance;
    a.out = output;
    a.C = c;
    a.H = h;
    a.W = w;
    a.N = n;
    a.OH = (h + 2 - 3) / stride + 1;
    a.OW = (w + 2 - 3) / stride + 1;
    a.bn = batch_normalize ? 1 : 0;
    a.tiles_x = (a.OW + CG_TC - 1) / CG_TC;
    const dn_f2 s = dn_split(slope);
    a.slope_hi = s.hi;
    a.slope_lo = s.lo;
    const dim3 grid((unsigned)(a.tiles_x * ((a.OH + CG_TR - 1) / CG_TR)), (unsigned)groups, (unsigned)batch);
    const int cg = c / groups;
    if (cg == 4 && stride == 1)
        hipLaunchKernelGGL((conv_group_kernel<4, 1>), grid, dim3(CG_THREADS), 0, dn_stream(), a);
    else if (cg == 4)
        hipLaunchKernelGGL((conv_group_kernel<4, 2>), grid, dim3(CG_THREADS), 0, dn_stream(), a);
    else
        hipLaunchKernelGGL((conv_group_kernel<8, 1>), grid, dim3(CG_THREADS), 0, dn_stream(), a);
    dn_check_launch("conv_group_forward");
}
