/*
 * conv_direct.hip - direct (non-GEMM) convolution with the fused batch-norm/bias/activation
 * tail.  Correct for every size / stride / pad / groups.  It serves two purposes:
 *   - grouped convolutions (ResNeXt 3x3 with 4..32 channels per group), whose per-group GEMMs
 *     are far too small for matrix-core tiles and are bound by HBM traffic instead;
 *   - the in-library cross-check of the MFMA kernel (conv_set_algo(1)).
 *
 * Work split: one workgroup handles DN_FPB consecutive filters of one group for a strip of
 * 256 output pixels of one image.  The strip's weights (DN_FPB x K) sit in LDS and are read as
 * wave-uniform broadcasts; each lane owns one output pixel, so input reads are coalesced along
 * the row and each loaded input value is reused for DN_FPB filters from a register.
 */
#include <hip/hip_runtime.h>

#include "device_math.h"
#include "hip.h"

#define DN_FPB 4          /* filters per workgroup */
#define DN_DIRECT_BLOCK 256
#define DN_DIRECT_KMAX 2048 /* per-filter weights kept in LDS per pass (floats) */

static inline hipStream_t dn_stream() { return (hipStream_t)hip_get_stream(); }

struct direct_args {
    const float *in;
    const float *w;
    const float *biases, *scales, *mean, *var;
    float *out;
    int batch, c, h, wd, n, groups, size, stride, pad, oh, ow, bn, act;
};

__global__ __launch_bounds__(DN_DIRECT_BLOCK) void conv_direct_kernel(direct_args a)
{
    __shared__ float wsm[DN_FPB * DN_DIRECT_KMAX];
    const int cg = a.c / a.groups;
    const int ng = a.n / a.groups;
    const int K = cg * a.size * a.size;
    const int P = a.oh * a.ow;
    const int fblocks_per_group = (ng + DN_FPB - 1) / DN_FPB;
    const int g = blockIdx.y / fblocks_per_group;
    const int f0 = g * ng + (blockIdx.y % fblocks_per_group) * DN_FPB; /* first filter */
    const int nf = min(DN_FPB, g * ng + ng - f0);
    const int b = blockIdx.z;
    const int p = blockIdx.x * DN_DIRECT_BLOCK + threadIdx.x;
    const bool live = p < P;
    const int oy = live ? p / a.ow : 0;
    const int ox = live ? p % a.ow : 0;
    const int iy0 = oy * a.stride - a.pad;
    const int ix0 = ox * a.stride - a.pad;
    const float *img = a.in + ((long)b * a.c + (long)g * cg) * a.h * a.wd;

    /* batch-norm constants of the workgroup's filters, once per workgroup (a double square root
     * and division each); visible to all threads after the first barrier of the K loop */
    __shared__ dn_bn_row rows[DN_FPB];
    if ((int)threadIdx.x < nf) {
        const int f = f0 + threadIdx.x;
        rows[threadIdx.x] = dn_bn_make(a.bn, a.biases[f], a.bn ? a.scales[f] : 1.f, a.bn ? a.mean[f] : 0.f,
                                       a.bn ? a.var[f] : 1.f);
    }

    float acc[DN_FPB];
#pragma unroll
    for (int j = 0; j < DN_FPB; ++j) acc[j] = 0.f;

    const int ss = a.size * a.size;
    for (int k0 = 0; k0 < K; k0 += DN_DIRECT_KMAX) {
        const int kc = min(DN_DIRECT_KMAX, K - k0);
        __syncthreads();
        for (int i = threadIdx.x; i < DN_FPB * kc; i += DN_DIRECT_BLOCK) {
            const int j = i / kc, k = i % kc;
            wsm[j * DN_DIRECT_KMAX + k] = (j < nf) ? a.w[(long)(f0 + j) * K + k0 + k] : 0.f;
        }
        __syncthreads();
        if (live) {
            for (int k = 0; k < kc; ++k) {
                const int kk = k0 + k;
                const int ci = kk / ss;
                const int r = kk - ci * ss;
                const int ky = r / a.size;
                const int kx = r - ky * a.size;
                const int iy = iy0 + ky, ix = ix0 + kx;
                float v = 0.f;
                if (iy >= 0 && iy < a.h && ix >= 0 && ix < a.wd) v = img[((long)ci * a.h + iy) * a.wd + ix];
#pragma unroll
                for (int j = 0; j < DN_FPB; ++j) acc[j] = fmaf(wsm[j * DN_DIRECT_KMAX + k], v, acc[j]);
            }
        }
    }
    if (!live) return;
#pragma unroll
    for (int j = 0; j < DN_FPB; ++j) {
        if (j >= nf) continue;
        const int f = f0 + j;
        const float y = dn_activate(dn_bn_apply(acc[j], rows[j], a.bn), a.act);
        a.out[((long)b * a.n + f) * P + p] = y;
    }
}

extern "C" void conv_direct_forward(const float *input, const float *weights, const float *biases,
                                    const float *scales, const float *rolling_mean,
                                    const float *rolling_variance, float *output, int batch, int c,
                                    int h, int w, int n, int groups, int size, int stride, int pad,
                                    int batch_normalize, int activation)
{
    direct_args a;
    a.in = input;
    a.w = weights;
    a.biases = biases;
    a.scales = scales;
    a.mean = rolling_mean;
    a.var = rolling_variance;
    a.out = output;
    a.batch = batch;
    a.c = c;
    a.h = h;
    a.wd = w;
    a.n = n;
    a.groups = groups;
    a.size = size;
    a.stride = stride;
    a.pad = pad;
    a.oh = (h + 2 * pad - size) / stride + 1;
    a.ow = (w + 2 * pad - size) / stride + 1;
    a.bn = batch_normalize ? 1 : 0;
    a.act = activation;
    const int ng = n / groups;
    const int fblocks = groups * ((ng + DN_FPB - 1) / DN_FPB);
    const int P = a.oh * a.ow;
    if (fblocks > 65535 || batch > 65535) dn_fatal("conv_direct_forward: grid too large");
    dim3 grid((P + DN_DIRECT_BLOCK - 1) / DN_DIRECT_BLOCK, fblocks, batch);
    hipLaunchKernelGGL(conv_direct_kernel, grid, dim3(DN_DIRECT_BLOCK), 0, dn_stream(), a);
    dn_check_launch("conv_direct_forward");
}
