/*
 * local.hip - the locally connected layer of the yolov1 networks (forward_local_layer,
 * src/local_layer.c:91-120; forward_local_layer_gpu :186-215 runs the same loop with one
 * cuBLAS call per location).
 *
 * A convolution whose filters are not shared between output positions: location j has its own
 * [n][size*size*c] weight matrix, stored location-major (src/local_layer.c:107), and a bias per
 * output element (src/local_layer.c:98).  With every weight used once per image the layer streams
 * its weights from HBM (462 MB for yolov1's 7x7x256 layer on 3x3x1024 patches), so the kernel is
 * laid out around that stream: the patches of every location are gathered once into a work
 * buffer; a workgroup then owns one location, 16 filters and 16 images (4 filters and 4 images
 * for batches up to 4), copies the patches into LDS chunk by chunk of k, and uses every weight
 * that arrives for all its images.  Lanes run along k, so a wave's weight loads are contiguous
 * rows.  A connected layer at a small batch is the one-location case of the same stream
 * (forward_connected_stream_gpu below).
 * Sums are formed in a fixed order (per lane along k, then a butterfly over the lanes), so
 * the result is the same from run to run.
 */
#include <hip/hip_runtime.h>

#include "device_math.h"
#include "hip.h"

#define LC_THREADS 256

static inline hipStream_t dn_stream() { return (hipStream_t)hip_get_stream(); }

struct local_args {
    const float *in, *weights, *biases, *patches;
    float *out;
    int batch, c, h, w, n, size, stride, pad, oh, ow, K, act;
};

/* Step 1: the patches, once per layer call: patches[location][image][k] with k = (channel, ky, kx)
 * as im2col_cpu orders its rows and zero outside the image (src/im2col.c:3-38).  Reads are short
 * scattered runs out of an input that sits in L2; writes are contiguous. */
__global__ void local_patches_kernel(local_args a, float *patches)
{
    const long total = (long)a.oh * a.ow * a.batch * a.K;
    const int ss = a.size * a.size;
    const long chw = (long)a.c * a.h * a.w;
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const int k = (int)(i % a.K);
        const long t = i / a.K;
        const int b = (int)(t % a.batch);
        const int j = (int)(t / a.batch);
        const int oy = j / a.ow, ox = j - oy * a.ow;
        const int ci = k / ss;
        const int r = k - ci * ss;
        const int ky = r / a.size;
        const int kx = r - ky * a.size;
        const int iy = oy * a.stride + ky - a.pad;
        const int ix = ox * a.stride + kx - a.pad;
        float v = 0.f;
        if (iy >= 0 && iy < a.h && ix >= 0 && ix < a.w) v = a.in[b * chw + ((long)ci * a.h + iy) * a.w + ix];
        patches[i] = v;
    }
}

/* Step 2.  A workgroup owns one location, 4*FW filters and NB images; four waves, FW filters each,
 * lanes along k.  Per chunk of KC values of k the NB patches are copied into LDS and every
 * weight that arrives from memory is used for all NB images (16 images, 4 filters per wave and
 * chunks of 256; 4 images, 1 filter per wave and chunks of 1024 for small batches).  Both sets of loads of a chunk are
 * issued before the first barrier, so a chunk costs one memory round trip, which the other
 * workgroups of the CU fill with their arithmetic.  Image groups of one (location, filters) pair
 * are neighbours in the grid, so their common weights are fetched from HBM once and served to the
 * other groups by the memory-side cache. */
template <int LC_NB, int LC_FW, int LC_KC>
__global__ __launch_bounds__(LC_THREADS, 4) void local_kernel(local_args a, int image_groups)
{
    static_assert(LC_NB * LC_FW <= 64, "one lane per (filter, image) pair in the final reduction");
    static_assert(LC_KC % LC_THREADS == 0, "every thread copies the same number of patch columns");
    __shared__ float tile[LC_NB][LC_KC];
    const int j = blockIdx.x / image_groups;
    const int b0 = (blockIdx.x - j * image_groups) * LC_NB;
    const int lane = threadIdx.x & 63;
    const int f0 = blockIdx.y * (LC_THREADS / 64 * LC_FW) + (threadIdx.x >> 6) * LC_FW;
    const int locations = a.oh * a.ow;

    const float *wrow[LC_FW];
#pragma unroll
    for (int i = 0; i < LC_FW; ++i) {
        const int f = f0 + i < a.n ? f0 + i : a.n - 1; /* rows past the last filter repeat it; never stored */
        wrow[i] = a.weights + ((long)j * a.n + f) * a.K;
    }
    const float *prow = a.patches + ((long)j * a.batch + b0) * a.K;
    float acc[LC_FW][LC_NB];
#pragma unroll
    for (int i = 0; i < LC_FW; ++i)
#pragma unroll
        for (int b = 0; b < LC_NB; ++b) acc[i][b] = 0.f;

    /* Workgroups start at different chunks of K: rows of the weight matrix lie a multiple of 4 KB
     * apart for the usual channel counts, so workgroups that all began at k = 0 would walk the
     * same few memory channels in step (measured: 2.5x slower). */
    const int nchunks = (a.K + LC_KC - 1) / LC_KC;
    const int rot = (int)((j * 5u + blockIdx.y * 3u) % (unsigned)nchunks);
    for (int step = 0; step < nchunks; ++step) {
        const int chunk = step + rot < nchunks ? step + rot : step + rot - nchunks;
        const int k0 = chunk * LC_KC;
        /* the chunk's weights (KC/64 per filter and lane); past the end of K the patch is zero in LDS,
         * the weight is read from a clamped address and replaced by zero */
        float wv[LC_KC / 64][LC_FW];
#pragma unroll
        for (int t = 0; t < LC_KC / 64; ++t) {
            const int k = k0 + lane + 64 * t;
            const int kc = k < a.K ? k : a.K - 1;
#pragma unroll
            for (int i = 0; i < LC_FW; ++i) {
                const float v = wrow[i][kc];
                wv[t][i] = k < a.K ? v : 0.f;
            }
        }
        /* the chunk's patches: thread t copies columns t, t+256, ... of each image's row */
        float pv[LC_KC / LC_THREADS][LC_NB];
#pragma unroll
        for (int h = 0; h < LC_KC / LC_THREADS; ++h) {
            const int k = k0 + threadIdx.x + h * LC_THREADS;
#pragma unroll
            for (int b = 0; b < LC_NB; ++b)
                pv[h][b] = (b0 + b < a.batch && k < a.K) ? prow[(long)b * a.K + k] : 0.f;
        }
        __syncthreads(); /* the previous chunk has been consumed */
#pragma unroll
        for (int h = 0; h < LC_KC / LC_THREADS; ++h)
#pragma unroll
            for (int b = 0; b < LC_NB; ++b) tile[b][threadIdx.x + h * LC_THREADS] = pv[h][b];
        __syncthreads();
#pragma unroll
        for (int t = 0; t < LC_KC / 64; ++t) {
#pragma unroll
            for (int b = 0; b < LC_NB; ++b) {
                const float x = tile[b][lane + 64 * t];
#pragma unroll
                for (int i = 0; i < LC_FW; ++i) acc[i][b] = fmaf(wv[t][i], x, acc[i][b]);
            }
        }
    }

    /* butterfly over the 64 lanes; lane i*16+b keeps the sum of filter i, image b */
    float mine = 0.f;
#pragma unroll
    for (int i = 0; i < LC_FW; ++i)
#pragma unroll
        for (int b = 0; b < LC_NB; ++b) {
            float v = acc[i][b];
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
            if (lane == i * LC_NB + b) mine = v;
        }
    const int f = f0 + lane / LC_NB;
    const int b = b0 + lane % LC_NB;
    if (lane < LC_NB * LC_FW && f < a.n && b < a.batch) {
        const long o = ((long)b * a.n + f) * locations + j;
        a.out[o] = dn_activate(a.biases[(long)f * locations + j] + mine, a.act);
    }
}

static float *g_patches = 0; /* patches of the current call, grown on demand and kept */
static size_t g_patches_floats = 0;
static long g_patch_budget = 1L << 28; /* floats (1 GiB): larger batches run in slices of images */

extern "C" void local_set_patch_budget(long floats)
{
    if (floats < 1) dn_fatal("local_set_patch_budget: the budget must be positive");
    g_patch_budget = floats;
}

/* The reference sizes its output with local_out_height / _width (src/local_layer.c:10-24: h - size
 * without padding, h - 1 with it) but fills its column buffer with im2col_cpu, whose own count is
 * (h + 2*pad - size)/stride + 1.  The two agree for the shapes the layer is used with (pad 0, or
 * size 3 with pad 1); where they differ the reference reads columns its im2col never wrote, so
 * such a geometry is refused here. */
extern "C" void forward_local_gpu(const float *input, const float *weights, const float *biases, float *output,
                                  int batch, int c, int h, int w, int n, int size, int stride, int pad,
                                  int activation)
{
    if (batch < 1 || c < 1 || h < 1 || w < 1 || n < 1 || size < 1 || stride < 1 || pad < 0)
        dn_fatal("forward_local_gpu: bad geometry");
    if (activation < 0 || activation > DN_SELU) dn_fatal("forward_local_gpu: unknown activation");
    const int oh = (h - (pad ? 1 : size)) / stride + 1;
    const int ow = (w - (pad ? 1 : size)) / stride + 1;
    if (oh < 1 || ow < 1 || (pad ? 1 : size) > h || (pad ? 1 : size) > w) dn_fatal("forward_local_gpu: empty output");
    if ((h + 2 * pad - size) / stride + 1 != oh || (w + 2 * pad - size) / stride + 1 != ow)
        dn_fatal("forward_local_gpu: pad and size give im2col a different output size than the layer's");
    if ((long)c * size * size >= (1L << 31) || (long)oh * ow > 0x7fffffffL) dn_fatal("forward_local_gpu: too large");
    const long K = (long)c * size * size;
    const long per_image = (long)oh * ow * K;
    if (per_image > g_patch_budget) dn_fatal("forward_local_gpu: one image's patches exceed the work buffer's budget");
    const int slice = (int)(g_patch_budget / per_image < batch ? g_patch_budget / per_image : batch);
    const size_t need = (size_t)per_image * slice;
    if (need > g_patches_floats) {
        if (g_patches) hip_free(g_patches);
        g_patches = hip_make_array(0, need);
        g_patches_floats = need;
    }
    for (int first = 0; first < batch; first += slice) {
        local_args a;
        a.batch = batch - first < slice ? batch - first : slice;
        a.in = input + (long)first * c * h * w;
        a.out = output + (long)first * n * oh * ow;
        a.weights = weights;
        a.biases = biases;
        a.patches = g_patches;
        a.c = c;
        a.h = h;
        a.w = w;
        a.n = n;
        a.size = size;
        a.stride = stride;
        a.pad = pad;
        a.oh = oh;
        a.ow = ow;
        a.K = (int)K;
        a.act = activation;
        const long total = per_image * a.batch;
        const long pb = (total + 255) / 256;
        hipLaunchKernelGGL(local_patches_kernel, dim3((unsigned)(pb > 65536 ? 65536 : pb)), dim3(256), 0, dn_stream(), a,
                           g_patches);
        const bool few = a.batch <= 4; /* one filter per wave, 4 images, 1024-wide chunks: more bytes in flight */
        const int fpb = LC_THREADS / 64 * (few ? 1 : 4);
        const int groups = few ? 1 : (a.batch + 15) / 16;
        if ((long)oh * ow * groups > 0x7fffffffL) dn_fatal("forward_local_gpu: too many locations x images for one launch");
        dim3 grid((unsigned)(oh * ow * groups), (unsigned)((n + fpb - 1) / fpb));
        if (grid.y > 65535u) dn_fatal("forward_local_gpu: too many filters for one launch");
        if (few)
            hipLaunchKernelGGL((local_kernel<4, 1, 1024>), grid, dim3(LC_THREADS), 0, dn_stream(), a, groups);
        else
            hipLaunchKernelGGL((local_kernel<16, 4, 256>), grid, dim3(LC_THREADS), 0, dn_stream(), a, groups);
    }
    dn_check_launch("forward_local_gpu");
}

/* A connected layer without batch-norm at a small batch is the same weight stream with a single
 * location whose "patches" are the layer's input rows themselves: forward_connected_layer
 * (src/connected_layer.c:140-167: gemm, add_bias, activate) as one pass over the weights.  One
 * filter per wave keeps outputs/4 workgroups in flight (1024 for a 4096-wide layer); up to 4 images
 * share a weight in registers, up to 16 through the wider tile. */
extern "C" void forward_connected_stream_gpu(const float *input, const float *weights, const float *biases,
                                             float *output, int batch, int inputs, int outputs, int activation)
{
    if (batch < 1 || inputs < 1 || outputs < 1) dn_fatal("forward_connected_stream_gpu: bad geometry");
    if (activation < 0 || activation > DN_SELU) dn_fatal("forward_connected_stream_gpu: unknown activation");
    local_args a;
    a.in = input;
    a.patches = input;
    a.weights = weights;
    a.biases = biases;
    a.out = output;
    a.batch = batch;
    a.c = inputs;
    a.h = a.w = a.size = a.stride = a.oh = a.ow = 1;
    a.pad = 0;
    a.n = outputs;
    a.K = inputs;
    a.act = activation;
    const int nb = batch <= 4 ? 4 : 16;
    const int fpb = LC_THREADS / 64 * (nb == 4 ? 1 : 2);
    const int groups = (batch + nb - 1) / nb;
    dim3 grid((unsigned)groups, (unsigned)((outputs + fpb - 1) / fpb));
    if (grid.y > 65535u) dn_fatal("forward_connected_stream_gpu: too many outputs for one launch");
    if (nb == 4)
        hipLaunchKernelGGL((local_kernel<4, 1, 1024>), grid, dim3(LC_THREADS), 0, dn_stream(), a, groups);
    else
        hipLaunchKernelGGL((local_kernel<16, 2, 512>), grid, dim3(LC_THREADS), 0, dn_stream(), a, groups);
    dn_check_launch("forward_connected_stream_gpu");
}
