/*
 * pool.hip - maxpool (+argmax), global average pool, softmax, and the stand-alone im2col.
 * maxpool and im2col are pure index work and must be bit-exact; avgpool and softmax are
 * wavefront reductions (64 lanes, DPP-free shuffles via __shfl_xor).
 */
#include <hip/hip_runtime.h>
#include <float.h>
#include <stdint.h>

#include "device_math.h"
#include "hip.h"

#define DN_BLOCK 256

static inline hipStream_t dn_stream() { return (hipStream_t)hip_get_stream(); }

static inline int dn_blocks(long n)
{
    long b = (n + DN_BLOCK - 1) / DN_BLOCK;
    if (b < 1) b = 1;
    const long cap = 256L * 32;
    return (int)(b > cap ? cap : b);
}

/* ---- maxpool ----------------------------------------------------------------------------- */
/* One thread per output.  Window cells are visited in row-major order and only a strictly
 * larger value replaces the running maximum, so ties keep the first cell, and NaN never wins
 * (src/maxpool_layer.c:94-106).  Cells outside the image count as -FLT_MAX. */
template <bool WRITE_INDEX>
__global__ void maxpool_kernel(const float *in, float *out, int *indexes, long n, int c, int h, int w,
                               int oh, int ow, int size, int stride, int off)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        const int ox = (int)(i % ow);
        long t = i / ow;
        const int oy = (int)(t % oh);
        const long plane = t / oh; /* b*c + k */
        const float *src = in + plane * h * w;
        float best = -FLT_MAX;
        int best_i = -1;
        for (int dy = 0; dy < size; ++dy) {
            const int iy = off + oy * stride + dy;
            for (int dx = 0; dx < size; ++dx) {
                const int ix = off + ox * stride + dx;
                const bool inside = iy >= 0 && iy < h && ix >= 0 && ix < w;
                const float v = inside ? src[iy * w + ix] : -FLT_MAX;
                if (v > best) {
                    best = v;
                    best_i = (int)(plane * h * w) + iy * w + ix;
                }
            }
        }
        out[i] = best;
        if (WRITE_INDEX) indexes[i] = best_i;
    }
}

/* 2x2 stride-2 window that never leaves the image (every downsampling pool of the yolo
 * family): each thread makes two outputs from two 16-byte row reads. */
template <bool WRITE_INDEX>
__global__ void maxpool_2x2s2_kernel(const float4 *in, float2 *out, int2 *indexes, long npairs,
                                     int h, int w /* input */, int ow2 /* ow/2 */)
{
    const int w4 = w / 4;
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < npairs; i += (long)gridDim.x * blockDim.x) {
        const int xp = (int)(i % ow2);
        const long orow = i / ow2;          /* plane*oh + oy */
        const long irow = orow * 2;         /* plane*h + 2*oy, because h == 2*oh */
        const float4 a = in[irow * w4 + xp];
        const float4 b = in[(irow + 1) * w4 + xp];
        const int base = (int)(irow * w) + xp * 4;
        float m0 = -FLT_MAX, m1 = -FLT_MAX;
        int i0 = -1, i1 = -1;
        if (a.x > m0) { m0 = a.x; i0 = base; }
        if (a.y > m0) { m0 = a.y; i0 = base + 1; }
        if (b.x > m0) { m0 = b.x; i0 = base + w; }
        if (b.y > m0) { m0 = b.y; i0 = base + w + 1; }
        if (a.z > m1) { m1 = a.z; i1 = base + 2; }
        if (a.w > m1) { m1 = a.w; i1 = base + 3; }
        if (b.z > m1) { m1 = b.z; i1 = base + w + 2; }
        if (b.w > m1) { m1 = b.w; i1 = base + w + 3; }
        out[i] = make_float2(m0, m1);
        if (WRITE_INDEX) indexes[i] = make_int2(i0, i1);
    }
}

extern "C" void forward_maxpool_gpu(const float *input, float *output, int *indexes, int batch, int c,
                                    int h, int w, int size, int stride, int pad)
{
    if (batch <= 0 || c <= 0 || h <= 0 || w <= 0 || size <= 0 || stride <= 0 || pad < 0)
        dn_fatal("forward_maxpool_gpu: bad geometry");
    const int oh = (h + pad - size) / stride + 1;
    const int ow = (w + pad - size) / stride + 1;
    if (oh <= 0 || ow <= 0) dn_fatal("forward_maxpool_gpu: empty output");
    if ((long)batch * c * h * w > 0x7fffffffL) dn_fatal("forward_maxpool_gpu: input too large for int indexes");
    const long n = (long)batch * c * oh * ow;
    const int off = -pad / 2;
    const bool fast = size == 2 && stride == 2 && off == 0 && (w % 4) == 0 && (h % 2) == 0 &&
                      oh * 2 == h && ow * 2 == w && ((uintptr_t)input & 15) == 0 &&
                      ((uintptr_t)output & 7) == 0 && (!indexes || ((uintptr_t)indexes & 7) == 0);
    if (fast) {
        const long npairs = n / 2;
        if (indexes)
            hipLaunchKernelGGL((maxpool_2x2s2_kernel<true>), dim3(dn_blocks(npairs)), dim3(DN_BLOCK), 0,
                               dn_stream(), (const float4 *)input, (float2 *)output, (int2 *)indexes,
                               npairs, h, w, ow / 2);
        else
            hipLaunchKernelGGL((maxpool_2x2s2_kernel<false>), dim3(dn_blocks(npairs)), dim3(DN_BLOCK), 0,
                               dn_stream(), (const float4 *)input, (float2 *)output, (int2 *)0, npairs, h,
                               w, ow / 2);
    } else {
        if (indexes)
            hipLaunchKernelGGL((maxpool_kernel<true>), dim3(dn_blocks(n)), dim3(DN_BLOCK), 0, dn_stream(),
                               input, output, indexes, n, c, h, w, oh, ow, size, stride, off);
        else
            hipLaunchKernelGGL((maxpool_kernel<false>), dim3(dn_blocks(n)), dim3(DN_BLOCK), 0, dn_stream(),
                               input, output, (int *)0, n, c, h, w, oh, ow, size, stride, off);
    }
    dn_check_launch("forward_maxpool_gpu");
}

/* ---- wavefront reductions ---------------------------------------------------------------- */
__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

/* ---- global average pool: one wavefront per (b, k) plane --------------------------------- */
__global__ void avgpool_kernel(const float *in, float *out, int planes, int area)
{
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int lane = threadIdx.x & 63;
    if (wave >= planes) return;
    const float *p = in + (long)wave * area;
    float s = 0;
    for (int i = lane; i < area; i += 64) s += p[i];
    s = wave_sum(s);
    if (lane == 0) out[wave] = s / (float)area;
}

extern "C" void forward_avgpool_gpu(const float *input, float *output, int batch, int c, int h, int w)
{
    if (batch <= 0 || c <= 0 || h <= 0 || w <= 0) dn_fatal("forward_avgpool_gpu: bad geometry");
    const int planes = batch * c;
    const int waves_per_block = DN_BLOCK / 64;
    hipLaunchKernelGGL(avgpool_kernel, dim3((planes + waves_per_block - 1) / waves_per_block),
                       dim3(DN_BLOCK), 0, dn_stream(), input, output, planes, h * w);
    dn_check_launch("forward_avgpool_gpu");
}

/* ---- softmax: one wavefront per (b, group) row ------------------------------------------- */
__global__ void softmax_kernel(const float *in, float *out, int n, int rows, int groups, int batch_offset,
                               int group_offset, int stride, float temp)
{
    const int row = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int lane = threadIdx.x & 63;
    if (row >= rows) return;
    const int b = row / groups, g = row % groups;
    const float *x = in + (long)b * batch_offset + (long)g * group_offset;
    float *y = out + (long)b * batch_offset + (long)g * group_offset;
    float largest = -FLT_MAX;
    for (int i = lane; i < n; i += 64) largest = fmaxf(largest, x[(long)i * stride]);
    largest = wave_max(largest);
    const float lt = largest / temp;
    float sum = 0;
    for (int i = lane; i < n; i += 64) {
        const float arg = __fsub_rn(x[(long)i * stride] / temp, lt);
        const float e = (float)exp((double)arg);
        sum += e;
        y[(long)i * stride] = e;
    }
    sum = wave_sum(sum);
    for (int i = lane; i < n; i += 64) y[(long)i * stride] = y[(long)i * stride] / sum;
}

extern "C" void softmax_gpu(float *input, int n, int batch, int batch_offset, int groups, int group_offset,
                            int stride, float temp, float *output)
{
    if (n <= 0 || batch <= 0 || groups <= 0) dn_fatal("softmax_gpu: bad geometry");
    if (input == output) dn_fatal("softmax_gpu: in-place operation is not supported");
    const int rows = batch * groups;
    const int waves_per_block = DN_BLOCK / 64;
    hipLaunchKernelGGL(softmax_kernel, dim3((rows + waves_per_block - 1) / waves_per_block), dim3(DN_BLOCK),
                       0, dn_stream(), (const float *)input, output, n, rows, groups, batch_offset,
                       group_offset, stride, temp);
    dn_check_launch("softmax_gpu");
}

/* ---- im2col: the column matrix the reference's GEMM consumes (src/im2col.c:16-39).  The
 * convolution kernels never materialise it; this entry point exists for callers that want the
 * matrix itself and as the bit-exact check of the gather index map. ------------------------ */
__global__ void im2col_kernel(const float *im, float *col, long n, int height, int width, int ksize,
                              int stride, int pad, int oh, int ow)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        const int ox = (int)(i % ow);
        long t = i / ow;
        const int oy = (int)(t % oh);
        const int r = (int)(t / oh); /* row of the column matrix: (ch*ksize + ky)*ksize + kx */
        const int kx = r % ksize;
        const int ky = (r / ksize) % ksize;
        const int ch = r / (ksize * ksize);
        const int iy = oy * stride + ky - pad;
        const int ix = ox * stride + kx - pad;
        float v = 0.f;
        if (iy >= 0 && ix >= 0 && iy < height && ix < width) v = im[ix + (long)width * (iy + (long)height * ch)];
        col[i] = v;
    }
}

extern "C" void im2col_gpu(float *im, int channels, int height, int width, int ksize, int stride, int pad,
                           float *data_col)
{
    if (channels <= 0 || height <= 0 || width <= 0 || ksize <= 0 || stride <= 0 || pad < 0)
        dn_fatal("im2col_gpu: bad geometry");
    const int oh = (height + 2 * pad - ksize) / stride + 1;
    const int ow = (width + 2 * pad - ksize) / stride + 1;
    if (oh <= 0 || ow <= 0) dn_fatal("im2col_gpu: empty output");
    const long n = (long)channels * ksize * ksize * oh * ow;
    hipLaunchKernelGGL(im2col_kernel, dim3(dn_blocks(n)), dim3(DN_BLOCK), 0, dn_stream(), (const float *)im,
                       data_col, n, height, width, ksize, stride, pad, oh, ow);
    dn_check_launch("im2col_gpu");
}
