/*
 * conv_mfma.hip - implicit-GEMM convolution on the CDNA4 matrix cores (fp32 MFMA), with the
 * batch-norm / bias / activation tail fused into the epilogue.
 *
 * GEMM view (per layer, groups == 1):   Out[M x N] = W[M x K] * Col[K x N]
 *   M = filters, K = size*size*c in the reference's (channel, ky, kx) order,
 *   N = batch*out_h*out_w; the batch folds into N, each image's output slab [M][out_h*out_w] is
 *   contiguous exactly as the reference lays it out (src/convolutional_layer.c:458-465).
 * The column matrix is never written to memory: each workgroup gathers its K-chunk of Col
 * straight from the NCHW input (the index map of src/im2col.c:26-35) into LDS.
 *
 * Tiling (64-wide wavefronts, 4 waves per workgroup):
 *   workgroup tile BM x BN x 16; wave tile WM x WN built from 32x32 accumulators of
 *   v_mfma_f32_32x32x2_f32 (TM x TN of them).  LDS holds A as [BM][16+4] and B as [BN][16+4]
 *   floats (k contiguous, 16-byte padded rows), double buffered; one ds_read_b128 per operand
 *   row feeds four MFMA k-steps.  Within a 16-wide chunk the k index a lane uses at step s of
 *   half hb is hb*8 + (lane/32)*4 + s for A and B alike, a bijection of the chunk, so the
 *   result is the plain sum over k.
 *   Global loads for chunk i+1 are issued before the MFMAs of chunk i and land in LDS after
 *   them (one barrier per chunk).
 * Weights are pre-packed to [K/16][Mpad][16] (zero padded, Mpad multiple of 128) so the A tile
 * is one contiguous, 16-byte aligned block for any BM.
 * Workgroup ids are remapped so that the tiles sharing a slice of the input run on the same
 * XCD (ids are dealt round-robin over the 8 XCDs, each with its own L2).
 */
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "device_math.h"
#include "hip.h"

typedef float f32x16 __attribute__((ext_vector_type(16)));

#define DN_BK 16
#define DN_LDK 20 /* padded LDS row, floats */
#define DN_MPAD 128
#define DN_THREADS 256

static inline hipStream_t dn_stream() { return (hipStream_t)hip_get_stream(); }

extern "C" void conv_direct_forward(const float *, const float *, const float *, const float *,
                                    const float *, const float *, float *, int, int, int, int, int,
                                    int, int, int, int, int, int);

struct mfma_args {
    const float *in;
    const float *wp; /* packed weights */
    const float *biases, *scales, *mean, *var;
    float *out;
    int C, H, W, M, K, KCH, Mpad;
    int P, OW;          /* out_h*out_w, out_w */
    long Ntotal;        /* batch * P */
    int stride, pad, size;
    int bn, act;
    int tiles_m, tiles_n, per_xcd;
};

/* k -> (channel, ky, kx) for a size x size kernel in the reference's im2col row order. */
template <int KS>
__device__ __forceinline__ void split_k(int k, int size, int &ci, int &ky, int &kx)
{
    if (KS == 1) {
        ci = k;
        ky = 0;
        kx = 0;
    } else if (KS == 3) {
        ci = (k * 7282) >> 16; /* k/9 for k < 32768 */
        const int r = k - ci * 9;
        ky = (r * 11) >> 5;    /* r/3 for r < 9 */
        kx = r - ky * 3;
    } else {
        const int ss = size * size;
        ci = k / ss;
        const int r = k - ci * ss;
        ky = r / size;
        kx = r - ky * size;
    }
}

template <int BM, int BN, int WM, int WN, int KS>
__global__ __launch_bounds__(DN_THREADS) void conv_mfma_kernel(mfma_args a)
{
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int WAVES_N = BN / WN;
    static_assert((BM / WM) * (BN / WN) == 4, "four waves per workgroup");
    constexpr int A_F4 = (BM * 4 + DN_THREADS - 1) / DN_THREADS; /* float4 loads of A per thread */
    constexpr int B_G = BN / 64;                                  /* 4-k groups of B per thread */

    __shared__ __attribute__((aligned(16))) float As[2][BM * DN_LDK];
    __shared__ __attribute__((aligned(16))) float Bs[2][BN * DN_LDK];
    __shared__ dn_bn_row rows[BM];

    /* XCD-aware tile order: workgroup id -> (xcd, slot) -> linear tile with tile_m fastest. */
    const int bid = blockIdx.x;
    const int lin = (bid & 7) * a.per_xcd + (bid >> 3);
    if (lin >= a.tiles_m * a.tiles_n) return;
    const int tile_m = lin % a.tiles_m;
    const int tile_n = lin / a.tiles_m;
    const int m0 = tile_m * BM;
    const long n0 = (long)tile_n * BN;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave / WAVES_N) * WM;
    const int wn0 = (wave % WAVES_N) * WN;

    /* per-filter batch-norm constants of this tile */
    for (int i = tid; i < BM; i += DN_THREADS) {
        const int m = m0 + i;
        dn_bn_row r = dn_bn_make(0, 0.f, 1.f, 0.f, 1.f);
        if (m < a.M)
            r = dn_bn_make(a.bn, a.biases[m], a.bn ? a.scales[m] : 1.f, a.bn ? a.mean[m] : 0.f,
                           a.bn ? a.var[m] : 1.f);
        rows[i] = r;
    }

    /* ---- gather bookkeeping: this thread's output pixel for the B tile ---- */
    const int bn_local = tid % BN;              /* column of the tile this thread gathers */
    const int kq0 = __builtin_amdgcn_readfirstlane(tid / BN); /* first 4-k group (wave-uniform) */
    constexpr int KQ_STEP = DN_THREADS / BN;    /* distance between this thread's groups */
    const long ncol = n0 + bn_local;
    const bool col_ok = ncol < a.Ntotal;
    int iy0 = 0, ix0 = 0;
    long pix_base = 0;
    {
        const long nn = col_ok ? ncol : 0;
        const int b = (int)(nn / a.P);
        const int p = (int)(nn - (long)b * a.P);
        const int oy = p / a.OW;
        const int ox = p - oy * a.OW;
        iy0 = oy * a.stride - a.pad;
        ix0 = ox * a.stride - a.pad;
        pix_base = (long)b * a.C * a.H * a.W + (long)iy0 * a.W + ix0;
    }
    const int HW = a.H * a.W;

    float4 a_reg[A_F4];
    float b_reg[B_G][4];

    auto load_chunk = [&](int kc) {
        /* A: contiguous block of BM*16 floats */
        const float4 *src = (const float4 *)(a.wp + ((long)kc * a.Mpad + m0) * DN_BK);
#pragma unroll
        for (int i = 0; i < A_F4; ++i) {
            const int idx = tid + i * DN_THREADS;
            if (BM * 4 >= DN_THREADS || idx < BM * 4) a_reg[i] = src[idx];
        }
        /* B: gathered */
#pragma unroll
        for (int g = 0; g < B_G; ++g) {
            const int kbase = kc * DN_BK + (kq0 + g * KQ_STEP) * 4;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int k = kbase + j;
                int ci, ky, kx;
                split_k<KS>(k, a.size, ci, ky, kx);
                float v = 0.f;
                if (KS == 1) {
                    if (col_ok && k < a.K) v = a.in[pix_base + (long)ci * HW];
                } else {
                    const int iy = iy0 + ky, ix = ix0 + kx;
                    const bool ok = col_ok && k < a.K && (unsigned)iy < (unsigned)a.H &&
                                    (unsigned)ix < (unsigned)a.W;
                    if (ok) v = a.in[pix_base + (long)ci * HW + ky * a.W + kx];
                }
                b_reg[g][j] = v;
            }
        }
    };

    auto store_chunk = [&](int buf) {
#pragma unroll
        for (int i = 0; i < A_F4; ++i) {
            const int idx = tid + i * DN_THREADS;
            if (BM * 4 >= DN_THREADS || idx < BM * 4) {
                const int row = idx >> 2, kq = idx & 3;
                *(float4 *)&As[buf][row * DN_LDK + kq * 4] = a_reg[i];
            }
        }
#pragma unroll
        for (int g = 0; g < B_G; ++g) {
            const int kq = kq0 + g * KQ_STEP;
            *(float4 *)&Bs[buf][bn_local * DN_LDK + kq * 4] =
                make_float4(b_reg[g][0], b_reg[g][1], b_reg[g][2], b_reg[g][3]);
        }
    };

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int li = lane & 31; /* row of A / column of B inside a 32x32 block */
    const int kh = lane >> 5; /* which half of the k pair this lane feeds */

    load_chunk(0);
    store_chunk(0);
    __syncthreads();

    for (int kc = 0; kc < a.KCH; ++kc) {
        const int buf = kc & 1;
        const bool more = kc + 1 < a.KCH;
        if (more) load_chunk(kc + 1);
#pragma unroll
        for (int hb = 0; hb < 2; ++hb) {
            float4 av[TM], bv[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i)
                av[i] = *(const float4 *)&As[buf][(wm0 + i * 32 + li) * DN_LDK + hb * 8 + kh * 4];
#pragma unroll
            for (int j = 0; j < TN; ++j)
                bv[j] = *(const float4 *)&Bs[buf][(wn0 + j * 32 + li) * DN_LDK + hb * 8 + kh * 4];
#pragma unroll
            for (int s = 0; s < 4; ++s) {
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    const float ae = s == 0 ? av[i].x : s == 1 ? av[i].y : s == 2 ? av[i].z : av[i].w;
#pragma unroll
                    for (int j = 0; j < TN; ++j) {
                        const float be = s == 0 ? bv[j].x : s == 1 ? bv[j].y : s == 2 ? bv[j].z : bv[j].w;
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(ae, be, acc[i][j], 0, 0, 0);
                    }
                }
            }
        }
        if (more) store_chunk(buf ^ 1);
        __syncthreads();
    }

    /* ---- epilogue: accumulator register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4 and
     * column l%32 of its 32x32 block ---- */
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const long n = n0 + wn0 + j * 32 + li;
        if (n >= a.Ntotal) continue;
        const int b = (int)(n / a.P);
        const int p = (int)(n - (long)b * a.P);
        float *obase = a.out + (long)b * a.M * a.P + p;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int ml = wm0 + i * 32 + 8 * (r >> 2) + 4 * kh + (r & 3);
                const int m = m0 + ml;
                if (m >= a.M) continue;
                const float y = dn_bn_apply(acc[i][j][r], rows[ml], a.bn);
                float z;
                if (a.act == DN_LEAKY) z = dn_activate_t<DN_LEAKY>(y);
                else if (a.act == DN_LINEAR) z = y;
                else z = dn_activate(y, a.act);
                obase[(long)m * a.P] = z;
            }
        }
    }
}

/* ---- weight packing ---------------------------------------------------------------------- */
__global__ void pack_weights_kernel(const float *w, float *packed, int M, int K, int Mpad, long total)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const int kk = (int)(i % DN_BK);
        long t = i / DN_BK;
        const int m = (int)(t % Mpad);
        const int kc = (int)(t / Mpad);
        const int k = kc * DN_BK + kk;
        packed[i] = (m < M && k < K) ? w[(long)m * K + k] : 0.f;
    }
}

extern "C" size_t conv_packed_floats(int n, int c, int groups, int size)
{
    if (groups != 1) return 0;
    const long K = (long)c * size * size;
    const long kch = (K + DN_BK - 1) / DN_BK;
    const long mpad = ((long)n + DN_MPAD - 1) / DN_MPAD * DN_MPAD;
    return (size_t)(kch * mpad * DN_BK);
}

extern "C" void conv_pack_weights_gpu(const float *weights, float *packed, int n, int c, int groups, int size)
{
    const size_t total = conv_packed_floats(n, c, groups, size);
    if (!total) return;
    const int K = c * size * size;
    const int mpad = (n + DN_MPAD - 1) / DN_MPAD * DN_MPAD;
    long blocks = (long)((total + 255) / 256);
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(pack_weights_kernel, dim3((int)blocks), dim3(256), 0, dn_stream(), weights, packed, n,
                       K, mpad, (long)total);
    dn_check_launch("conv_pack_weights_gpu");
}

/* ---- dispatch ---------------------------------------------------------------------------- */
static int g_algo = 0;
extern "C" void conv_set_algo(int algo) { g_algo = algo; }

static float *g_scratch = 0;       /* per-call repack buffer for callers without a packed copy */
static size_t g_scratch_floats = 0;

template <int BM, int BN, int WM, int WN>
static void launch_tile(const mfma_args &a0, int ks)
{
    mfma_args a = a0;
    a.tiles_m = (a.M + BM - 1) / BM;
    a.tiles_n = (int)((a.Ntotal + BN - 1) / BN);
    const long total = (long)a.tiles_m * a.tiles_n;
    a.per_xcd = (int)((total + 7) / 8);
    const dim3 grid((unsigned)(a.per_xcd * 8));
    if (ks == 1)
        hipLaunchKernelGGL((conv_mfma_kernel<BM, BN, WM, WN, 1>), grid, dim3(DN_THREADS), 0, dn_stream(), a);
    else if (ks == 3)
        hipLaunchKernelGGL((conv_mfma_kernel<BM, BN, WM, WN, 3>), grid, dim3(DN_THREADS), 0, dn_stream(), a);
    else
        hipLaunchKernelGGL((conv_mfma_kernel<BM, BN, WM, WN, 0>), grid, dim3(DN_THREADS), 0, dn_stream(), a);
}

extern "C" void forward_convolutional_gpu(const float *input, const float *weights, const float *packed,
                                          const float *biases, const float *scales,
                                          const float *rolling_mean, const float *rolling_variance,
                                          float *output, int batch, int c, int h, int w, int n,
                                          int groups, int size, int stride, int pad,
                                          int batch_normalize, int activation)
{
    if (batch <= 0 || c <= 0 || h <= 0 || w <= 0 || n <= 0 || groups <= 0 || size <= 0 || stride <= 0 || pad < 0)
        dn_fatal("forward_convolutional_gpu: bad geometry");
    if (c % groups || n % groups) dn_fatal("forward_convolutional_gpu: groups must divide channels and filters");
    if (activation < 0 || activation > DN_SELU) dn_fatal("forward_convolutional_gpu: unknown activation");
    if (!input || !weights || !biases || !output) dn_fatal("forward_convolutional_gpu: null pointer");
    if (batch_normalize && (!scales || !rolling_mean || !rolling_variance))
        dn_fatal("forward_convolutional_gpu: batch_normalize needs scales, rolling_mean, rolling_variance");
    if (size == 1 && (stride != 1 || pad != 0))
        dn_fatal("forward_convolutional_gpu: a 1x1 kernel needs stride 1 and pad 0");
    const int oh = (h + 2 * pad - size) / stride + 1;
    const int ow = (w + 2 * pad - size) / stride + 1;
    if (oh <= 0 || ow <= 0) dn_fatal("forward_convolutional_gpu: empty output");
    if ((long)batch * c * h * w >= (1L << 40) || (long)batch * n * oh * ow >= (1L << 40))
        dn_fatal("forward_convolutional_gpu: tensor too large");

    const long K = (long)(c / groups) * size * size;
    if (groups != 1 || g_algo == 1 || (size == 3 && K >= 32768)) {
        conv_direct_forward(input, weights, biases, scales, rolling_mean, rolling_variance, output, batch, c,
                            h, w, n, groups, size, stride, pad, batch_normalize, activation);
        return;
    }

    if (!packed) {
        const size_t need = conv_packed_floats(n, c, groups, size);
        if (need > g_scratch_floats) {
            if (g_scratch) hip_free(g_scratch);
            g_scratch = hip_make_array(0, need);
            g_scratch_floats = need;
        }
        conv_pack_weights_gpu(weights, g_scratch, n, c, groups, size);
        packed = g_scratch;
    }

    mfma_args a;
    a.in = input;
    a.wp = packed;
    a.biases = biases;
    a.scales = scales;
    a.mean = rolling_mean;
    a.var = rolling_variance;
    a.out = output;
    a.C = c;
    a.H = h;
    a.W = w;
    a.M = n;
    a.K = (int)K;
    a.KCH = (int)((K + DN_BK - 1) / DN_BK);
    a.Mpad = (n + DN_MPAD - 1) / DN_MPAD * DN_MPAD;
    a.P = oh * ow;
    a.OW = ow;
    a.Ntotal = (long)batch * a.P;
    a.stride = stride;
    a.pad = pad;
    a.size = size;
    a.bn = batch_normalize ? 1 : 0;
    a.act = activation;
    a.tiles_m = a.tiles_n = a.per_xcd = 0;
    const int ks = size == 1 ? 1 : size == 3 ? 3 : 0;
    if (n <= 32)
        launch_tile<32, 256, 32, 64>(a, ks);
    else if (n <= 64)
        launch_tile<64, 256, 64, 64>(a, ks);
    else
        launch_tile<128, 128, 64, 64>(a, ks);
    dn_check_launch("forward_convolutional_gpu");
}
