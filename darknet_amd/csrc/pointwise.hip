/*
 * pointwise.hip - the memory-bound element-wise kernels of the darknet forward path:
 * fill / copy / activate / normalize / scale / bias / shortcut / upsample / route / yolo /
 * binarize.  All are HBM-bound: one coalesced read of each operand, one coalesced write,
 * 16-byte accesses where the geometry allows it, grid-stride over a launch that covers the
 * 256 CUs several times.
 */
#include <hip/hip_runtime.h>
#include <float.h>
#include <stdint.h>

#include "device_math.h"
#include "hip.h"

#define DN_BLOCK 256

static inline hipStream_t dn_stream() { return (hipStream_t)hip_get_stream(); }

static inline int dn_blocks(long n, int per_thread = 1)
{
    long b = (n + (long)DN_BLOCK * per_thread - 1) / ((long)DN_BLOCK * per_thread);
    if (b < 1) b = 1;
    const long cap = 256L * 32; /* 32 resident-ish blocks per CU worth of grid-stride */
    return (int)(b > cap ? cap : b);
}

static inline bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

/* ---------------------------------------------------------------------------------------- */
__global__ void fill_kernel(long n, float alpha, float *x, int incx)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        x[i * incx] = alpha;
}

__global__ void fill4_kernel(long n4, float alpha, float4 *x)
{
    const float4 v = make_float4(alpha, alpha, alpha, alpha);
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n4; i += (long)gridDim.x * blockDim.x)
        x[i] = v;
}

extern "C" void fill_gpu(int N, float ALPHA, float *X, int INCX)
{
    if (N <= 0) return;
    if (INCX == 1 && aligned16(X) && (N & 3) == 0) {
        hipLaunchKernelGGL(fill4_kernel, dim3(dn_blocks(N / 4)), dim3(DN_BLOCK), 0, dn_stream(),
                           (long)N / 4, ALPHA, (float4 *)X);
    } else {
        hipLaunchKernelGGL(fill_kernel, dim3(dn_blocks(N)), dim3(DN_BLOCK), 0, dn_stream(),
                           (long)N, ALPHA, X, INCX);
    }
    dn_check_launch("fill_gpu");
}

__global__ void copy_kernel(long n, const float *x, long offx, int incx, float *y, long offy, int incy)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        y[offy + i * incy] = x[offx + i * incx];
}

__global__ void copy4_kernel(long n4, const float4 *x, float4 *y)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n4; i += (long)gridDim.x * blockDim.x)
        y[i] = x[i];
}

extern "C" void copy_gpu_offset(int N, float *X, int OFFX, int INCX, float *Y, int OFFY, int INCY)
{
    if (N <= 0) return;
    const float *xs = X + OFFX;
    float *ys = Y + OFFY;
    if (INCX == 1 && INCY == 1 && aligned16(xs) && aligned16(ys) && (N & 3) == 0) {
        hipLaunchKernelGGL(copy4_kernel, dim3(dn_blocks(N / 4)), dim3(DN_BLOCK), 0, dn_stream(),
                           (long)N / 4, (const float4 *)xs, (float4 *)ys);
    } else {
        hipLaunchKernelGGL(copy_kernel, dim3(dn_blocks(N)), dim3(DN_BLOCK), 0, dn_stream(),
                           (long)N, (const float *)X, (long)OFFX, INCX, Y, (long)OFFY, INCY);
    }
    dn_check_launch("copy_gpu");
}

extern "C" void copy_gpu(int N, float *X, int INCX, float *Y, int INCY)
{
    copy_gpu_offset(N, X, 0, INCX, Y, 0, INCY);
}

/* ---------------------------------------------------------------------------------------- */
__global__ void activate_kernel(float *x, long n, int a)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        x[i] = dn_activate(x[i], a);
}

__global__ void activate4_kernel(float4 *x, long n4, int a)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n4; i += (long)gridDim.x * blockDim.x) {
        float4 v = x[i];
        v.x = dn_activate(v.x, a);
        v.y = dn_activate(v.y, a);
        v.z = dn_activate(v.z, a);
        v.w = dn_activate(v.w, a);
        x[i] = v;
    }
}

/* activate_array_gpu for tensors of any length (internal: the convolution uses it for the
 * activations its epilogue does not carry) */
extern "C" void dn_activate_array(float *x, long n, int activation)
{
    if (n <= 0 || activation == DN_LINEAR) return;
    if (activation < 0 || activation > DN_SELU) dn_fatal("activate_array_gpu: unknown activation");
    if (aligned16(x) && (n & 3) == 0) {
        hipLaunchKernelGGL(activate4_kernel, dim3(dn_blocks(n / 4)), dim3(DN_BLOCK), 0, dn_stream(),
                           (float4 *)x, n / 4, activation);
    } else {
        hipLaunchKernelGGL(activate_kernel, dim3(dn_blocks(n)), dim3(DN_BLOCK), 0, dn_stream(), x, n,
                           activation);
    }
    dn_check_launch("activate_array_gpu");
}

extern "C" void activate_array_gpu(float *x, int n, int activation) { dn_activate_array(x, (long)n, activation); }

/* ---- batch-norm pieces as separate passes (the fused convolution does not use them; they are
 * the reference-named helpers for callers that still run the chain step by step) ----------- */
__global__ void normalize_kernel(float *x, const float *mean, const float *variance, long n,
                                 int filters, int spatial)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        const int f = (int)((i / spatial) % filters);
        const double inv = 1.0 / (sqrt((double)variance[f]) + (double).000001f);
        x[i] = (float)((double)__fsub_rn(x[i], mean[f]) * inv);
    }
}

__global__ void scale_bias_kernel(float *x, const float *scales, long n, int filters, int spatial)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        x[i] = __fmul_rn(x[i], scales[(i / spatial) % filters]);
}

__global__ void add_bias_kernel(float *x, const float *biases, long n, int filters, int spatial)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        x[i] = __fadd_rn(x[i], biases[(i / spatial) % filters]);
}

extern "C" void normalize_gpu(float *x, float *mean, float *variance, int batch, int filters, int spatial)
{
    const long n = (long)batch * filters * spatial;
    if (n <= 0) return;
    hipLaunchKernelGGL(normalize_kernel, dim3(dn_blocks(n)), dim3(DN_BLOCK), 0, dn_stream(), x, mean,
                       variance, n, filters, spatial);
    dn_check_launch("normalize_gpu");
}

extern "C" void scale_bias_gpu(float *output, float *scales, int batch, int n, int size)
{
    const long total = (long)batch * n * size;
    if (total <= 0) return;
    hipLaunchKernelGGL(scale_bias_kernel, dim3(dn_blocks(total)), dim3(DN_BLOCK), 0, dn_stream(),
                       output, scales, total, n, size);
    dn_check_launch("scale_bias_gpu");
}

extern "C" void add_bias_gpu(float *output, float *biases, int batch, int n, int size)
{
    const long total = (long)batch * n * size;
    if (total <= 0) return;
    hipLaunchKernelGGL(add_bias_kernel, dim3(dn_blocks(total)), dim3(DN_BLOCK), 0, dn_stream(),
                       output, biases, total, n, size);
    dn_check_launch("add_bias_gpu");
}

/* The inference branch of a standalone [batchnorm] layer (src/batchnorm_layer.c:191-192,231-234;
 * CPU form :135-155) in one pass: out = ((in - mean) / (sqrt(var) + 1e-6f)) * scale + bias with a
 * rounding to float after each step, as the reference's copy / normalize / scale_bias / add_bias
 * passes round. */
__global__ void batchnorm_kernel(const float *in, float *out, const float *scales, const float *biases,
                                 const float *mean, const float *variance, long n, int filters, int spatial)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        const int f = (int)((i / spatial) % filters);
        const dn_bn_row r = dn_bn_make(1, biases[f], scales[f], mean[f], variance[f]);
        out[i] = dn_bn_apply(in[i], r, 1);
    }
}

extern "C" void forward_batchnorm_gpu(const float *input, float *output, const float *scales, const float *biases,
                                      const float *rolling_mean, const float *rolling_variance, int batch,
                                      int c, int spatial)
{
    const long n = (long)batch * c * spatial;
    if (n <= 0) return;
    if (!input || !output || !scales || !biases || !rolling_mean || !rolling_variance)
        dn_fatal("forward_batchnorm_gpu: null pointer");
    hipLaunchKernelGGL(batchnorm_kernel, dim3(dn_blocks(n)), dim3(DN_BLOCK), 0, dn_stream(), input, output,
                       scales, biases, rolling_mean, rolling_variance, n, c, spatial);
    dn_check_launch("forward_batchnorm_gpu");
}

/* cuda_random (src/cuda.c:106-118): n uniform floats in (0, 1], as curandGenerateUniform fills them.
 * The reference seeds its generator with time(0), so the values were never reproducible there; the
 * stream here is a counter-based hash of (call number, index).  Only training-time dropout and
 * crop read it; inference never does. */
__global__ void random_kernel(float *x, long n, unsigned long long call)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        unsigned long long z = call * 0xD1342543DE82EF95ull + (unsigned long long)(i + 1) * 0x9E3779B97F4A7C15ull;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        z ^= z >> 31;
        x[i] = (float)((z >> 40) + 1) * (1.0f / 16777216.0f); /* 24 bits: (0, 1] */
    }
}

extern "C" void hip_random(float *x_gpu, size_t n)
{
    static unsigned long long calls = 0;
    if (!n) return;
    hip_require_device("cuda_random");
    hipLaunchKernelGGL(random_kernel, dim3(dn_blocks((long)n)), dim3(DN_BLOCK), 0, dn_stream(), x_gpu, (long)n, ++calls);
    dn_check_launch("cuda_random");
}

extern "C" void cuda_random(float *x_gpu, size_t n) { hip_random(x_gpu, n); }

/* ---- shortcut --------------------------------------------------------------------------- */
/* Same-geometry residual add (every shortcut of the darknet53 family): 16-byte accesses. */
__global__ void shortcut_same4_kernel(const float4 *in, const float4 *add, float4 *out, long n4,
                                      float s1, float s2, int a)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n4; i += (long)gridDim.x * blockDim.x) {
        const float4 x = in[i];
        const float4 y = add[i];
        float4 r;
        r.x = dn_activate(__fadd_rn(__fmul_rn(s1, x.x), __fmul_rn(s2, y.x)), a);
        r.y = dn_activate(__fadd_rn(__fmul_rn(s1, x.y), __fmul_rn(s2, y.y)), a);
        r.z = dn_activate(__fadd_rn(__fmul_rn(s1, x.z), __fmul_rn(s2, y.z)), a);
        r.w = dn_activate(__fadd_rn(__fmul_rn(s1, x.w), __fmul_rn(s2, y.w)), a);
        out[i] = r;
    }
}

/* General geometry: out indexed over (b, k, y, x) of the (w2,h2,c2) tensor. */
__global__ void shortcut_general_kernel(const float *in, const float *add, float *out, long n,
                                        int w1, int h1, int c1, int w2, int h2, int c2,
                                        int stride, int sample, int minw, int minh, int minc,
                                        float s1, float s2, int a)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        const int x = (int)(i % w2);
        long t = i / w2;
        const int y = (int)(t % h2);
        t /= h2;
        const int k = (int)(t % c2);
        const int b = (int)(t / c2);
        float v = in[i];
        const int xi = x / sample, yi = y / sample;
        if (k < minc && x % sample == 0 && y % sample == 0 && xi < minw && yi < minh) {
            const long ai = (long)xi * stride + (long)w1 * ((long)yi * stride + (long)h1 * (k + (long)c1 * b));
            v = __fadd_rn(__fmul_rn(s1, v), __fmul_rn(s2, add[ai]));
        }
        out[i] = dn_activate(v, a);
    }
}

/* The same, one output plane (image b, channel k) per blockIdx.x and 32-bit index arithmetic: the
 * residual adds of the first block of a ResNeXt stage (more channels out than in, with or without a
 * halved map) are launches of 50-200 MB in which the 64-bit divisions of the kernel above cost more
 * than the memory traffic.  Four consecutive pixels per thread where the plane allows 16-byte
 * accesses and the two maps have the same size. */
template <bool QUAD>
__global__ void shortcut_planes_kernel(const float *in, const float *add, float *out, int w1, int h1, int c1,
                                       int w2, int h2, int c2, int stride, int sample, int minw, int minh,
                                       int minc, float s1, float s2, int a)
{
    const int plane = blockIdx.x, b = plane / c2, k = plane - b * c2;
    const int hw2 = h2 * w2;
    const long obase = (long)plane * hw2;
    const bool has_add = k < minc;
    const long abase = ((long)b * c1 + k) * h1 * w1;
    if (QUAD) { /* stride == sample == 1, w1 == w2, h1 == h2, hw2 % 4 == 0 */
        for (int q = blockIdx.y * blockDim.x + threadIdx.x; q < hw2 / 4; q += gridDim.y * blockDim.x) {
            float4 v = *(const float4 *)(in + obase + 4 * q);
            if (has_add) {
                const float4 r = *(const float4 *)(add + abase + 4 * q);
                v.x = __fadd_rn(__fmul_rn(s1, v.x), __fmul_rn(s2, r.x));
                v.y = __fadd_rn(__fmul_rn(s1, v.y), __fmul_rn(s2, r.y));
                v.z = __fadd_rn(__fmul_rn(s1, v.z), __fmul_rn(s2, r.z));
                v.w = __fadd_rn(__fmul_rn(s1, v.w), __fmul_rn(s2, r.w));
            }
            v.x = dn_activate(v.x, a);
            v.y = dn_activate(v.y, a);
            v.z = dn_activate(v.z, a);
            v.w = dn_activate(v.w, a);
            *(float4 *)(out + obase + 4 * q) = v;
        }
    } else {
        for (int p = blockIdx.y * blockDim.x + threadIdx.x; p < hw2; p += gridDim.y * blockDim.x) {
            const int y = p / w2, x = p - y * w2;
            float v = in[obase + p];
            const int xi = x / sample, yi = y / sample;
            if (has_add && x - xi * sample == 0 && y - yi * sample == 0 && xi < minw && yi < minh)
                v = __fadd_rn(__fmul_rn(s1, v), __fmul_rn(s2, add[abase + (long)(yi * stride) * w1 + xi * stride]));
            out[obase + p] = dn_activate(v, a);
        }
    }
}

extern "C" void forward_shortcut_gpu(const float *in, const float *add, float *out, int batch, int w1,
                                     int h1, int c1, int w2, int h2, int c2, float s1, float s2,
                                     int activation)
{
    if (w1 <= 0 || h1 <= 0 || c1 <= 0 || w2 <= 0 || h2 <= 0 || c2 <= 0 || batch <= 0)
        dn_fatal("forward_shortcut_gpu: empty geometry");
    int stride = w1 / w2, sample = w2 / w1;
    if (stride != h1 / h2 || sample != h2 / h1)
        dn_fatal("forward_shortcut_gpu: width and height ratios differ");
    if (stride < 1) stride = 1;
    if (sample < 1) sample = 1;
    const int minw = w1 < w2 ? w1 : w2, minh = h1 < h2 ? h1 : h2, minc = c1 < c2 ? c1 : c2;
    const long n = (long)batch * c2 * h2 * w2;
    const bool same = (w1 == w2 && h1 == h2 && c1 == c2);
    if (same && (n & 3) == 0 && aligned16(in) && aligned16(add) && aligned16(out)) {
        hipLaunchKernelGGL(shortcut_same4_kernel, dim3(dn_blocks(n / 4)), dim3(DN_BLOCK), 0, dn_stream(),
                           (const float4 *)in, (const float4 *)add, (float4 *)out, n / 4, s1, s2,
                           activation);
    } else if ((long)h2 * w2 >= 512 && (long)batch * c2 < (1L << 31) && (long)h2 * w2 < (1L << 24) &&
               (long)h1 * w1 < (1L << 30)) {
        /* (planes of a few hundred pixels leave most of a workgroup idle: the flat kernel below is faster there -
         * 46 against 66 us on 1024 planes of 14 x 14 per image, batch 64) */
        const long hw2 = (long)h2 * w2;
        const bool quad = w1 == w2 && h1 == h2 && (hw2 & 3) == 0 && aligned16(in) && aligned16(add) && aligned16(out);
        const long per_plane = quad ? hw2 / 4 : hw2;
        /* about four elements (or quads) per thread: the small planes of the late stages would otherwise be
         * tens of thousands of workgroups of one element per thread */
        const dim3 grid((unsigned)(batch * c2), (unsigned)((per_plane + 4 * DN_BLOCK - 1) / (4 * DN_BLOCK)));
        if (quad)
            hipLaunchKernelGGL(shortcut_planes_kernel<true>, grid, dim3(DN_BLOCK), 0, dn_stream(), in, add, out, w1, h1,
                               c1, w2, h2, c2, stride, sample, minw, minh, minc, s1, s2, activation);
        else
            hipLaunchKernelGGL(shortcut_planes_kernel<false>, grid, dim3(DN_BLOCK), 0, dn_stream(), in, add, out, w1, h1,
                               c1, w2, h2, c2, stride, sample, minw, minh, minc, s1, s2, activation);
    } else {
        hipLaunchKernelGGL(shortcut_general_kernel, dim3(dn_blocks(n)), dim3(DN_BLOCK), 0, dn_stream(),
                           in, add, out, n, w1, h1, c1, w2, h2, c2, stride, sample, minw, minh, minc,
                           s1, s2, activation);
    }
    dn_check_launch("forward_shortcut_gpu");
}

extern "C" void shortcut_gpu(int batch, int w1, int h1, int c1, float *add, int w2, int h2, int c2,
                             float s1, float s2, float *out)
{
    forward_shortcut_gpu(out, add, out, batch, w1, h1, c1, w2, h2, c2, s1, s2, DN_LINEAR);
}

/* ---- upsample (nearest) ------------------------------------------------------------------ */
__global__ void upsample_kernel(const float *in, float *out, long n, int w, int h, int stride, float scale)
{
    const int ow = w * stride, oh = h * stride;
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        const int x = (int)(i % ow);
        long t = i / ow;
        const int y = (int)(t % oh);
        const long plane = t / oh; /* b*c + k */
        out[i] = __fmul_rn(scale, in[plane * h * w + (long)(y / stride) * w + x / stride]);
    }
}

/* stride 2, even alignment: each thread turns 2 inputs into a 16-byte store on two rows. */
__global__ void upsample2_kernel(const float2 *in, float4 *out, long npairs, int w2 /* w/2 */, int h, float scale)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < npairs; i += (long)gridDim.x * blockDim.x) {
        const int xp = (int)(i % w2);
        const long row = i / w2; /* plane*h + y */
        const float2 v = in[i];
        const float a = __fmul_rn(scale, v.x), b = __fmul_rn(scale, v.y);
        const float4 o = make_float4(a, a, b, b);
        const long orow = row * 2; /* output row index within plane-major layout: (plane*2h + 2y) */
        out[orow * w2 + xp] = o;
        out[(orow + 1) * w2 + xp] = o;
    }
}

/* stride 2, any width: a thread turns one input into two 8-byte stores (rows 2y and 2y + 1; the
 * output rows have an even length, so the pairs are aligned whenever the tensor is). */
__global__ void upsample2e_kernel(const float *in, float2 *out, long n, int w, float scale)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        const int x = (int)(i % w);
        const long row = i / w; /* plane*h + y */
        const float a = __fmul_rn(scale, in[i]);
        const float2 o = make_float2(a, a);
        out[(row * 2) * w + x] = o;
        out[(row * 2 + 1) * w + x] = o;
    }
}

extern "C" void upsample_gpu(float *in, int w, int h, int c, int batch, int stride, int forward,
                             float scale, float *out)
{
    if (!forward) dn_fatal("upsample_gpu: only the forward (non-reverse) direction is built");
    if (stride < 1 || w <= 0 || h <= 0 || c <= 0 || batch <= 0) dn_fatal("upsample_gpu: bad geometry");
    const long n = (long)batch * c * h * w * stride * stride;
    if (stride == 2 && (w & 1) == 0 && aligned16(out) && ((uintptr_t)in & 7) == 0) {
        const long npairs = (long)batch * c * h * (w / 2);
        hipLaunchKernelGGL(upsample2_kernel, dim3(dn_blocks(npairs)), dim3(DN_BLOCK), 0, dn_stream(),
                           (const float2 *)in, (float4 *)out, npairs, w / 2, h, scale);
    } else if (stride == 2 && ((uintptr_t)out & 7) == 0) {
        const long nin = (long)batch * c * h * w;
        hipLaunchKernelGGL(upsample2e_kernel, dim3(dn_blocks(nin)), dim3(DN_BLOCK), 0, dn_stream(),
                           (const float *)in, (float2 *)out, nin, w, scale);
    } else {
        hipLaunchKernelGGL(upsample_kernel, dim3(dn_blocks(n)), dim3(DN_BLOCK), 0, dn_stream(),
                           (const float *)in, out, n, w, h, stride, scale);
    }
    dn_check_launch("upsample_gpu");
}

/* ---- route: per-image concatenation of up to DN_ROUTE_MAX sources in one launch ---------- */
#define DN_ROUTE_MAX 8
struct route_args {
    const float *src[DN_ROUTE_MAX];
    int size[DN_ROUTE_MAX];   /* floats per image of each source */
    int start[DN_ROUTE_MAX];  /* offset of each source within an output image */
    int nsrc;
    int outputs;              /* floats per output image */
};

template <typename T, int V>
__global__ void route_kernel(route_args a, T *out, long total /* in units of V floats */)
{
    const int out_v = a.outputs / V;
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const int b = (int)(i / out_v);
        const int off = (int)(i % out_v) * V;
        int s = 0;
#pragma unroll
        for (int j = 1; j < DN_ROUTE_MAX; ++j)
            if (j < a.nsrc && off >= a.start[j]) s = j;
        const T *src = (const T *)(a.src[s] + (long)b * a.size[s] + (off - a.start[s]));
        out[i] = *src;
    }
}

extern "C" void forward_route_gpu(const float *const *srcs, const int *sizes, int nsrc, float *output,
                                  int batch)
{
    if (nsrc < 1 || nsrc > DN_ROUTE_MAX) dn_fatal("forward_route_gpu: between 1 and 8 sources are supported");
    route_args a;
    int off = 0;
    bool v4 = aligned16(output);
    for (int i = 0; i < DN_ROUTE_MAX; ++i) {
        a.src[i] = i < nsrc ? srcs[i] : 0;
        a.size[i] = i < nsrc ? sizes[i] : 0;
        a.start[i] = off;
        if (i < nsrc) {
            if (sizes[i] <= 0 || !srcs[i]) dn_fatal("forward_route_gpu: empty source");
            v4 = v4 && (sizes[i] & 3) == 0 && aligned16(srcs[i]);
            off += sizes[i];
        }
    }
    a.nsrc = nsrc;
    a.outputs = off;
    const long total = (long)batch * off;
    if (total <= 0) return;
    if (v4) {
        hipLaunchKernelGGL((route_kernel<float4, 4>), dim3(dn_blocks(total / 4)), dim3(DN_BLOCK), 0,
                           dn_stream(), a, (float4 *)output, total / 4);
    } else {
        hipLaunchKernelGGL((route_kernel<float, 1>), dim3(dn_blocks(total)), dim3(DN_BLOCK), 0,
                           dn_stream(), a, output, total);
    }
    dn_check_launch("forward_route_gpu");
}

/* ---- yolo head: copy + logistic on entries 0,1 and 4.. of each anchor -------------------- */
__global__ void yolo_kernel(const float *in, float *out, long n, int plane, int entries)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        const int e = (int)((i / plane) % entries);
        const float v = in[i];
        out[i] = (e == 2 || e == 3) ? v : dn_logistic_fast(v);
    }
}

/* plane a multiple of 4: a 16-byte quad never straddles two entries */
__global__ void yolo4_kernel(const float4 *in, float4 *out, long n4, int plane4, int entries)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n4; i += (long)gridDim.x * blockDim.x) {
        const int e = (int)((i / plane4) % entries);
        float4 v = in[i];
        if (e != 2 && e != 3) {
            v.x = dn_logistic_fast(v.x);
            v.y = dn_logistic_fast(v.y);
            v.z = dn_logistic_fast(v.z);
            v.w = dn_logistic_fast(v.w);
        }
        out[i] = v;
    }
}

extern "C" void forward_yolo_gpu(const float *input, float *output, int batch, int w, int h,
                                 int n_anchors, int classes)
{
    if (batch <= 0 || w <= 0 || h <= 0 || n_anchors <= 0 || classes < 0) dn_fatal("forward_yolo_gpu: bad geometry");
    const int entries = 4 + classes + 1;
    const long n = (long)batch * n_anchors * entries * w * h;
    if (((w * h) & 3) == 0 && aligned16(input) && aligned16(output))
        hipLaunchKernelGGL(yolo4_kernel, dim3(dn_blocks(n / 4)), dim3(DN_BLOCK), 0, dn_stream(),
                           (const float4 *)input, (float4 *)output, n / 4, w * h / 4, entries);
    else
        hipLaunchKernelGGL(yolo_kernel, dim3(dn_blocks(n)), dim3(DN_BLOCK), 0, dn_stream(), input, output,
                           n, w * h, entries);
    dn_check_launch("forward_yolo_gpu");
}

/* ---- binarize ---------------------------------------------------------------------------- */
__global__ void binarize_kernel(const float *x, long n, float *binary)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        binary[i] = (x[i] > 0) ? 1.f : -1.f;
}

extern "C" void binarize_gpu(float *x, int n, float *binary)
{
    if (n <= 0) return;
    hipLaunchKernelGGL(binarize_kernel, dim3(dn_blocks(n)), dim3(DN_BLOCK), 0, dn_stream(),
                       (const float *)x, (long)n, binary);
    dn_check_launch("binarize_gpu");
}

/* One thread per filter walks its weights in order, so the float sum of |w| is rounded exactly
 * as the sequential CPU loop rounds it (src/convolutional_layer.c:28-41).  Weight tensors are
 * small; this runs once per forward of an xnor layer. */
__global__ void binarize_weights_kernel(const float *weights, int n, int size, float *binary)
{
    const int f = blockIdx.x * blockDim.x + threadIdx.x;
    if (f >= n) return;
    const float *w = weights + (long)f * size;
    float mean = 0;
    for (int i = 0; i < size; ++i) mean = (float)((double)mean + fabs((double)w[i]));
    mean = mean / size;
    for (int i = 0; i < size; ++i) binary[(long)f * size + i] = (w[i] > 0) ? mean : -mean;
}

extern "C" void binarize_weights_gpu(float *weights, int n, int size, float *binary)
{
    if (n <= 0 || size <= 0) return;
    hipLaunchKernelGGL(binarize_weights_kernel, dim3((n + 63) / 64), dim3(64), 0, dn_stream(),
                       (const float *)weights, n, size, binary);
    dn_check_launch("binarize_weights_gpu");
}

/* ---- reorg / flatten / crop: pure index work, bit-exact ------------------------------------ */
/* reorg_cpu of src/blas.c:9-30 (same argument meaning as reorg_gpu, src/blas.h:73): thread i
 * walks the (b, k, j, i) space of the c x h x w tensor x is described with; `forward` copies
 * x[in_index] to out[out_index], otherwise out[in_index] = x[out_index]. */
__global__ void reorg_kernel(const float *x, float *out, long n, int w, int h, int c, int stride, int forward)
{
    const int out_c = c / (stride * stride);
    for (long id = blockIdx.x * (long)blockDim.x + threadIdx.x; id < n; id += (long)gridDim.x * blockDim.x) {
        const int i = (int)(id % w);
        long t = id / w;
        const int j = (int)(t % h);
        t /= h;
        const int k = (int)(t % c);
        const long b = t / c;
        const int c2 = k % out_c;
        const int offset = k / out_c;
        const int w2 = i * stride + offset % stride;
        const int h2 = j * stride + offset / stride;
        const long out_index = w2 + (long)w * stride * (h2 + (long)h * stride * (c2 + (long)out_c * b));
        if (forward) out[out_index] = x[id];
        else out[id] = x[out_index];
    }
}

extern "C" void reorg_gpu(float *x, int w, int h, int c, int batch, int stride, int forward, float *out)
{
    if (w <= 0 || h <= 0 || c <= 0 || batch <= 0 || stride <= 0) dn_fatal("reorg_gpu: bad geometry");
    if (c % (stride * stride)) dn_fatal("reorg_gpu: stride*stride must divide the channel count");
    const long n = (long)w * h * c * batch;
    hipLaunchKernelGGL(reorg_kernel, dim3(dn_blocks(n)), dim3(DN_BLOCK), 0, dn_stream(), x, out, n, w, h, c, stride,
                       forward);
    dn_check_launch("reorg_gpu");
}

/* flatten of src/blas.c:32-49, out of place: [b][layers][spatial] <-> [b][spatial][layers] */
__global__ void flatten_kernel(const float *x, float *out, long n, int spatial, int layers, int forward)
{
    for (long id = blockIdx.x * (long)blockDim.x + threadIdx.x; id < n; id += (long)gridDim.x * blockDim.x) {
        const int i = (int)(id % spatial);
        long t = id / spatial;
        const int cc = (int)(t % layers);
        const long b = t / layers;
        const long i1 = b * layers * spatial + (long)cc * spatial + i;
        const long i2 = b * layers * spatial + (long)i * layers + cc;
        if (forward) out[i2] = x[i1];
        else out[i1] = x[i2];
    }
}

extern "C" void flatten_gpu(float *x, int spatial, int layers, int batch, int forward, float *out)
{
    if (spatial <= 0 || layers <= 0 || batch <= 0) dn_fatal("flatten_gpu: bad geometry");
    const long n = (long)spatial * layers * batch;
    hipLaunchKernelGGL(flatten_kernel, dim3(dn_blocks(n)), dim3(DN_BLOCK), 0, dn_stream(), x, out, n, spatial,
                       layers, forward);
    dn_check_launch("flatten_gpu");
}

/* forward_crop_layer at inference (src/crop_layer.c:67-103 with net.train == 0): the centred
 * window, then value*scale + trans in two float roundings (scale 2, trans -1 unless noadjust) */
__global__ void crop_kernel(const float *in, float *out, long n, int c, int h, int w, int oh, int ow, int dh,
                            int dw, float scale, float trans)
{
    for (long id = blockIdx.x * (long)blockDim.x + threadIdx.x; id < n; id += (long)gridDim.x * blockDim.x) {
        const int j = (int)(id % ow);
        long t = id / ow;
        const int i = (int)(t % oh);
        const long plane = t / oh; /* b*c + k */
        out[id] = __fadd_rn(__fmul_rn(in[(j + dw) + (long)w * ((i + dh) + (long)h * plane)], scale), trans);
    }
}

extern "C" void forward_crop_gpu(const float *input, float *output, int batch, int c, int h, int w, int out_h,
                                 int out_w, int noadjust)
{
    if (batch <= 0 || c <= 0 || h <= 0 || w <= 0 || out_h <= 0 || out_w <= 0 || out_h > h || out_w > w)
        dn_fatal("forward_crop_gpu: bad geometry");
    const long n = (long)batch * c * out_h * out_w;
    hipLaunchKernelGGL(crop_kernel, dim3(dn_blocks(n)), dim3(DN_BLOCK), 0, dn_stream(), input, output, n, c, h, w,
                       out_h, out_w, (h - out_h) / 2, (w - out_w) / 2, noadjust ? 1.f : 2.f, noadjust ? 0.f : -1.f);
    dn_check_launch("forward_crop_gpu");
}

/* ---- region head (yolov2): src/region_layer.c:158-184, the inference part of the CPU build -- */
/* copy + logistic on x, y, on objectness unless `background`, on the classes unless a softmax
 * follows; layout [b][anchor][coords + 1 + classes][h][w] */
__global__ void region_kernel(const float *in, float *out, long n, int plane, int entries, int coords,
                              int background, int softmax)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        const int e = (int)((i / plane) % entries);
        const float v = in[i];
        const bool act = e < 2 || (e == coords && !background) || (e > coords && !softmax);
        out[i] = act ? dn_activate(v, DN_LOGISTIC) : v;
    }
}

/* softmax over the classes of one (image, anchor, cell): softmax_cpu with stride = plane
 * (src/blas.c:305-332), one thread per cell so that neighbouring threads read neighbouring
 * addresses and the float sum runs in the reference's order */
__global__ void region_softmax_kernel(const float *in, float *out, long rows, int plane, int entries, int first,
                                      int n)
{
    for (long r = blockIdx.x * (long)blockDim.x + threadIdx.x; r < rows; r += (long)gridDim.x * blockDim.x) {
        const long group = r / plane;
        const int cell = (int)(r - group * plane);
        const float *x = in + (group * entries + first) * plane + cell;
        float *y = out + (group * entries + first) * plane + cell;
        float largest = -FLT_MAX;
        for (int i = 0; i < n; ++i) {
            const float v = x[(long)i * plane];
            if (v > largest) largest = v;
        }
        float sum = 0;
        for (int i = 0; i < n; ++i) {
            const float e = (float)exp((double)__fsub_rn(x[(long)i * plane], largest)); /* temp == 1 */
            sum = __fadd_rn(sum, e);
            y[(long)i * plane] = e;
        }
        for (int i = 0; i < n; ++i) y[(long)i * plane] = __fdiv_rn(y[(long)i * plane], sum);
    }
}

extern "C" void forward_region_gpu(const float *input, float *output, int batch, int w, int h, int n_anchors,
                                   int classes, int coords, int background, int softmax)
{
    if (batch <= 0 || w <= 0 || h <= 0 || n_anchors <= 0 || classes < 0)
        dn_fatal("forward_region_gpu: bad geometry");
    /* with more than four coordinates the reference's two forwards disagree (its GPU form applies
     * the logistic to entries 4 .. coords-1, src/region_layer.c:450-453, its CPU form does not,
     * :164-173), and no cfg in the tree uses them */
    if (coords != 4) dn_fatal("forward_region_gpu: coords must be 4");
    if (input == output) dn_fatal("forward_region_gpu: in-place operation is not supported");
    const int entries = coords + classes + 1;
    const int plane = w * h;
    const long n = (long)batch * n_anchors * entries * plane;
    hipLaunchKernelGGL(region_kernel, dim3(dn_blocks(n)), dim3(DN_BLOCK), 0, dn_stream(), input, output, n, plane,
                       entries, coords, background, softmax);
    if (softmax && classes + background > 0) {
        const long rows = (long)batch * n_anchors * plane;
        hipLaunchKernelGGL(region_softmax_kernel, dim3(dn_blocks(rows)), dim3(DN_BLOCK), 0, dn_stream(), input,
                           output, rows, plane, entries, coords + !background, classes + background);
    }
    dn_check_launch("forward_region_gpu");
}
