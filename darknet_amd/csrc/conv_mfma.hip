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
 *   workgroup tile BM x BN x 16 (128x128; 64x256 / 32x256 for layers with few filters); wave
 *   tile WM x WN built from 32x32 accumulators of v_mfma_f32_32x32x2_f32 (TM x TN of them).
 *   LDS holds a chunk of A as [4 slots][BM][4 floats] and of B as [4 slots][BN][4 floats]
 *   (k = 4*slot + j), written by direct-to-LDS buffer loads and double buffered; one
 *   ds_read_b128 per operand row feeds four MFMA k-steps.  Within a 16-wide chunk the k index a
 *   lane uses at step s of half hb is 4*(2*hb + lane/32) + s for A and B alike, a bijection of
 *   the chunk, so the result is the plain sum over k.
 *   Global loads for chunk i+1 are issued before the MFMAs of chunk i and land in LDS after
 *   them (one barrier per chunk).
 * Weights are pre-packed to [K/16][4 slots][Mpad][4] (zero padded, Mpad multiple of 128) so a
 * wave-load of A is one contiguous kilobyte for any BM; a bf16 copy for the reduced-precision
 * variants follows in the same buffer.
 * The last partial round of tiles is cut along K into slices that park raw accumulators and are
 * summed in slice order by conv_reduce_kernel (deterministic).
 * Epilogue: batch-norm, bias and activation in the accumulator layout, a turn through LDS, then
 * 256-byte row stores; a same-geometry residual add (shortcut layer) can ride along.
 * Three opt-in variants of the same kernel run on the bf16 matrix cores (template parameter BF16,
 * conv_set_precision): operands rounded to bf16 (1: fp32 activation tiles converted in registers,
 * 2: 3x3 layers gathering from a staged bf16 copy of the input; both with bf16 weights, four LDS
 * stages and 256x128 tiles), and fp32 emulated with three bf16 pieces per operand (3).
 *
 * Order of K.  The sum over k does not care about the order as long as A and B agree, and the
 * packing step can permute K for free, so two orders are used:
 *   - "tap blocked" (1x1, and 3x3 with pad 1, when c % 16 == 0): k' = (cb*taps + tap)*16 + ci,
 *     channel c = cb*16 + ci.  A 16-wide chunk is then 16 channels of ONE kernel tap: the whole
 *     chunk shares one border test and one scalar base address (input + (cb*16*H*W + tap shift)),
 *     each of a thread's loads adds a loop-invariant scalar i*H*W and the thread's fixed 32-bit
 *     pixel offset, and the nine taps of a channel block follow each other so their input lines
 *     are still in the L1/L2 when the next tap asks for them.  The loads are buffer loads:
 *     lanes whose tap falls outside the image carry an out-of-range offset and get their zero
 *     from the hardware range check, so the gather costs no vector ALU work at all.
 *   - the reference's own (channel, ky, kx) order for everything else (first layer with 3
 *     channels, 7x7 stems, odd channel counts), with a per-element index split.
 * Workgroup ids are remapped so that the tiles sharing a slice of the input run on the same
 * XCD (ids are dealt round-robin over the 8 XCDs, each with its own L2).
 */
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "device_math.h"
#include "hip.h"

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

#define DN_BK 16
#define DN_MPAD 128
#define DN_THREADS 256

static inline hipStream_t dn_stream() { return (hipStream_t)hip_get_stream(); }

extern "C" void conv_direct_forward(const float *, const float *, const float *, const float *,
                                    const float *, const float *, float *, int, int, int, int, int,
                                    int, int, int, int, int, int);

/* conv_group.hip: grouped 3x3 layers of 4 or 8 channels per group, on the vector ALU */
extern "C" int conv_group_serves(int batch, int c, int h, int w, int n, int groups, int size, int stride, int pad);
extern "C" const char *conv_group_kernel_name(int c, int groups, int stride);
extern "C" void conv_group_forward(const float *input, const float *weights, const float *biases, const float *scales,
                                   const float *rolling_mean, const float *rolling_variance, float *output, int batch,
                                   int c, int h, int w, int n, int groups, int stride, int batch_normalize, double slope);
/* conv_first.hip: the kernel of 3-channel first layers */
extern "C" void conv_first_device_setup(void);
extern "C" int conv_first_serves(int batch, int c, int h, int w, int n, int groups, int size, int stride, int pad);
extern "C" const char *conv_first_kernel_name(int c, int n, int pooled, int h, int w);
extern "C" void conv_first_forward(const float *input, const float *weights, const float *biases, const float *scales,
                                   const float *rolling_mean, const float *rolling_variance, float *out, float *pool,
                                   unsigned *bits, int batch, int c, int h, int w, int n, int batch_normalize,
                                   double slope, int cus, void *start, void *stop);

struct mfma_args {
    const float *in;
    const float *wp; /* packed weights */
    const void *wp16; /* the bf16 copy of the packed weights (bf16-operand mode) */
    unsigned wp16_records;
    unsigned plane16; /* bytes of one bf16 copy; the mid and lo copies of the three-piece mode follow the first */
    int Mpad16;
    const void *in16; /* staged bf16 copy of the input, [image][C/8][H*W][8] (bf16 mode, 3x3 layers) */
    unsigned in16_records;
    const float *biases, *scales, *mean, *var;
    float *out;
    int C, H, W, M, K, KCH, Mpad;
    int P, OW;          /* out_h*out_w, out_w */
    long Ntotal;        /* batch * P */
    int stride, pad, size;
    int bn;
    float slope_hi, slope_lo; /* activation slope (conv_inline_activation) as hi + lo floats */
    float sum_slope_hi, sum_slope_lo;
    int tiles_m, tiles_n, per_xcd;
    /* tile order: the filter tiles are cut into tiles_m / m_group bands of m_group tiles; a band's
     * tiles come first in the linear order (filter tile fastest inside the band), so the
     * consecutive range an XCD owns reads one band's weights and a share of the columns */
    int m_group, band_tiles;
    unsigned in_records; /* bytes the gather may address: input + bias row */
    unsigned wp_records; /* bytes of the packed weights */
    /* K-split tail: tiles [0, whole_tiles) are computed in one piece by workgroups
     * [0, 8*per_xcd); every later workgroup j computes K-slice j % split of tile
     * whole_tiles + j / split and leaves raw accumulators in `partial` for the reduce kernel */
    int whole_tiles, split;
    float *partial;
    /* grouped layers (see conv_grouped_tile): every 32-filter tile reads its own 32 input
     * channels and its own block of packed weights; 0 for ordinary layers */
    int grouped;
    /* fused residual add (null = none): sum[i] = act2(s1*out[i] + s2*add[i]) over the same
     * geometry as out, the arithmetic of src/blas.c:36 followed by src/shortcut_layer.c:64 */
    const float *add;
    float *sum;
    float s1, s2;
    /* fused yolo head instead (add == null, sum = the yolo layer's output): sum[i] = out[i] on the
     * w and h entries of every anchor, logistic(out[i]) elsewhere (src/yolo_layer.c:132-148);
     * > 0 = entries per anchor (5 + classes) */
    int yolo_entries;
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
    } else if (KS == 7) { /* the 7x7 stems: constant divisors, a few multiplies instead of two 32-bit divisions per k */
        ci = k / 49;
        const int r = k - ci * 49;
        ky = r / 7;
        kx = r - ky * 7;
    } else {
        const int ss = size * size;
        ci = k / ss;
        const int r = k - ci * ss;
        ky = r / size;
        kx = r - ky * size;
    }
}

typedef float float4u __attribute__((ext_vector_type(4), aligned(4)));

/* The three activations the epilogue applies itself share one branch-free form,
 *     f(y) = y > 0 ? y : (float)(slope * (double)y)      (evaluated as conv_mul_f2 below),
 * with slope .1 for leaky (src/activations.h:39), 1 for linear and 0 for relu: for relu the
 * reference's x*(x>0) (src/activations.h:35) and 0.*x agree on every input including -0, the
 * infinities and NaN.  Any other activation runs as a second pass over the output. */
__host__ __device__ inline bool conv_inline_activation(int act, double *slope)
{
    if (act == DN_LEAKY) *slope = .1;
    else if (act == DN_LINEAR) *slope = 1.;
    else if (act == DN_RELU) *slope = 0.;
    else return false;
    return true;
}

/* A double constant as an unevaluated sum of two floats: x*hi + x*lo with one fused rounding,
 * fmaf(x, hi, x*lo), reproduces (float)((double)x * c) except when the exact product lies within
 * ~2^-48 (relative) of a float rounding boundary, at a third of the instruction cost of the
 * convert / multiply / convert sequence in double precision. */
struct conv_f2 {
    float hi, lo;
};

__host__ __device__ inline conv_f2 conv_split(double c)
{
    conv_f2 r;
    r.hi = (float)c;
    r.lo = (float)(c - (double)r.hi);
    return r;
}

__device__ __forceinline__ float conv_mul_f2(float x, conv_f2 c) { return fmaf(x, c.hi, __fmul_rn(x, c.lo)); }

__device__ __forceinline__ float conv_slope(float y, conv_f2 slope) { return (y > 0) ? y : conv_mul_f2(y, slope); }

/* Per-filter constants of the tail: normalize (src/blas.c:154, as a multiplication by the
 * reciprocal of the double denominator), scale, bias (src/batchnorm_layer.c:151-154), each step
 * rounded to float as the reference's separate passes do.  Without batch-norm the constants are
 * neutral (mean 0, reciprocal 1, scale 1) and change no bit. */
struct conv_row_t {
    conv_f2 inv;
    float mean, scale, bias;
};

__device__ __forceinline__ conv_row_t conv_row(const mfma_args &a, int m)
{
    conv_row_t r;
    r.bias = a.biases[m];
    if (a.bn) {
        r.inv = conv_split(1.0 / (sqrt((double)a.var[m]) + (double).000001f));
        r.mean = a.mean[m];
        r.scale = a.scales[m];
    } else {
        r.inv.hi = 1.f;
        r.inv.lo = 0.f;
        r.mean = 0.f;
        r.scale = 1.f;
    }
    return r;
}

__device__ __forceinline__ float conv_tail_one(float acc, const conv_row_t &row, conv_f2 slope)
{
    float x = conv_mul_f2(__fsub_rn(acc, row.mean), row.inv);
    x = __fadd_rn(__fmul_rn(x, row.scale), row.bias);
    return conv_slope(x, slope);
}

__device__ __forceinline__ float conv_residual_one(const mfma_args &a, float y, float r)
{
    return conv_slope(__fadd_rn(__fmul_rn(a.s1, y), __fmul_rn(a.s2, r)), conv_f2{a.sum_slope_hi, a.sum_slope_lo});
}

/* the yolo head's value for filter m */
__device__ __forceinline__ bool conv_yolo_keeps(const mfma_args &a, int m)
{
    const int e = m % a.yolo_entries;
    return e == 2 || e == 3;
}
__device__ __forceinline__ float conv_yolo_one(float y, bool keep) { return keep ? y : dn_logistic_fast(y); }

/* Batch-norm / bias / activation and the store.  The MFMAs are issued with the pixel tile as
 * the row operand and the filter tile as the column operand, so accumulator register r of lane l
 * holds filter (l % 32) and pixel 8*(r/4) + 4*(l/32) + r%4 of its 32x32 block: a lane owns one
 * filter per 32-row block, so its batch-norm constants are loaded once and the tail is applied
 * in that layout.  Stored from there, every lane of a store would hit a different output row
 * (64 separate 16-byte pieces per instruction, and the rate of such pieces, not bytes, is what
 * the memory pipeline limits).  The finished values therefore take a turn through LDS first:
 * each wave owns 8 KB of the (by now idle) operand buffers, holding 32 filters x 64 pixels with
 * the 16-byte quads of a row XOR-swizzled by the row number (conflict-free both ways), and
 * reads them back with 16 lanes per filter row: a store instruction then covers 4 rows of 256
 * contiguous bytes, and the residual of a fused shortcut is read the same way. */
template <int TM, int TN>
__device__ __forceinline__ void conv_epilogue(const mfma_args &a, f32x16 (&acc)[TM][TN], float *E,
                                              const conv_row_t *rows, int m0, long n0, int wm0, int wn0, int lane)
{
    static_assert(TN == 1 || TN == 2, "a wave's tile is 32 or 64 columns wide");
    constexpr int QN = 8 * TN;  /* quads of four pixels per filter row of the turn buffer */
    constexpr int RS = 32 * TN; /* its row stride in floats */
    constexpr int RG = 64 / QN; /* filter rows one read instruction covers (4 or 8) */
    const int li = lane & 31, kh = lane >> 5;
    const int q = lane & (QN - 1), fr = lane / QN; /* after the turn: quad of 4 pixels, row within a group of RG */
    const int P = a.P;
    const int Nt = (int)a.Ntotal;            /* Ntotal < 2^31 on this path */
    const int n = (int)n0 + wn0 + 4 * q;
    const int b = (int)((unsigned)n / (unsigned)P);
    const int p = n - b * P;
    const long off = (long)b * a.M * P + p;  /* image*M*P + pixel */
    const bool quad_ok = p + 3 < P;          /* the quad lies in one image (then n + 3 < Ntotal too) */
    const long wrap = (long)(a.M - 1) * P;   /* what the offset gains when the pixel index wraps */
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int mrow = m0 + wm0 + i * 32;
        const conv_row_t row = rows[wm0 + i * 32 + li]; /* computed once per workgroup */
#pragma unroll
        for (int j = 0; j < TN; ++j) {
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) {
                float4 o;
                o.x = conv_tail_one(acc[i][j][rg * 4 + 0], row, conv_f2{a.slope_hi, a.slope_lo});
                o.y = conv_tail_one(acc[i][j][rg * 4 + 1], row, conv_f2{a.slope_hi, a.slope_lo});
                o.z = conv_tail_one(acc[i][j][rg * 4 + 2], row, conv_f2{a.slope_hi, a.slope_lo});
                o.w = conv_tail_one(acc[i][j][rg * 4 + 3], row, conv_f2{a.slope_hi, a.slope_lo});
                const int qq = j * 8 + 2 * rg + kh;
                *(float4 *)&E[li * RS + ((qq ^ (li & (QN - 1))) << 2)] = o;
            }
        }
        __builtin_amdgcn_wave_barrier(); /* LDS operations of one wave complete in order */
#pragma unroll
        for (int t = 0; t < 32 / RG; ++t) {
            const int f = fr + RG * t;
            const float4 o = *(const float4 *)&E[f * RS + ((q ^ (f & (QN - 1))) << 2)];
            const int m = mrow + f;
            if (m >= a.M || n >= Nt) continue;
            const long o_off = off + (long)m * P;
            if (quad_ok) {
                *(float4u *)(a.out + o_off) = (float4u){o.x, o.y, o.z, o.w};
                if (a.yolo_entries) {
                    const bool keep = conv_yolo_keeps(a, m);
                    float4u s;
                    s.x = conv_yolo_one(o.x, keep);
                    s.y = conv_yolo_one(o.y, keep);
                    s.z = conv_yolo_one(o.z, keep);
                    s.w = conv_yolo_one(o.w, keep);
                    *(float4u *)(a.sum + o_off) = s;
                } else if (a.sum) {
                    const float4u r = *(const float4u *)(a.add + o_off);
                    float4u s;
                    s.x = conv_residual_one(a, o.x, r.x);
                    s.y = conv_residual_one(a, o.y, r.y);
                    s.z = conv_residual_one(a, o.z, r.z);
                    s.w = conv_residual_one(a, o.w, r.w);
                    *(float4u *)(a.sum + o_off) = s;
                }
            } else { /* image boundary or end of N inside the quad: element by element */
                const float v[4] = {o.x, o.y, o.z, o.w};
                int pc = p;
                long offc = o_off;
                for (int c = 0; c < 4 && n + c < Nt; ++c) {
                    while (pc >= P) {
                        pc -= P;
                        offc += wrap;
                    }
                    a.out[offc] = v[c];
                    if (a.yolo_entries)
                        a.sum[offc] = conv_yolo_one(v[c], conv_yolo_keeps(a, m));
                    else if (a.sum)
                        a.sum[offc] = conv_residual_one(a, v[c], a.add[offc]);
                    ++pc;
                    ++offc;
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
}

/* Sums the K-slices of one tail tile in slice order (deterministic) and applies the epilogue, for
 * one unit u of the tile: four accumulator registers of one lane (r = 4g .. 4g+3), i.e. four
 * consecutive pixels of one filter row (see conv_epilogue for the register map), so consecutive
 * units read consecutive dwords of every slice and the result leaves as one 16-byte store.
 * Units whose filter or pixels lie outside the layer read nothing. */
template <int BM, int BN, int WM, int WN>
__device__ __forceinline__ void conv_reduce_unit(const mfma_args &a, int t, int u)
{
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int WAVES_N = BN / WN;
    const int lin = a.whole_tiles + t;
    const int band = lin / a.band_tiles, in_band = lin - band * a.band_tiles;
    const int m0 = (band * a.m_group + in_band % a.m_group) * BM;
    const long n0 = (long)(in_band / a.m_group) * BN;
    /* u = ((wave*TM*TN + i*TN + j)*4 + g)*64 + lane */
    const int lane = u & 63;
    const int g = (u >> 6) & 3;
    int q = u >> 8;
    const int j = q % TN;
    q /= TN;
    const int i = q % TM;
    const int wave = q / TM;
    const int m = m0 + (wave / WAVES_N) * WM + i * 32 + (lane & 31);
    const long n = n0 + (wave % WAVES_N) * WN + j * 32 + 8 * g + 4 * (lane >> 5);
    if (m >= a.M || n >= a.Ntotal) return;
    /* element ((wave*TM*TN + i*TN + j)*16 + 4g + rr)*64 + lane of each slice */
    const float *ws = a.partial + (long)t * a.split * (BM * BN) + ((u >> 8) * 16 + 4 * g) * 64 + lane;
    float sum[4] = {0.f, 0.f, 0.f, 0.f};
    int sl = 0;
    /* four slices' loads in flight at a time; the additions keep slice order */
    for (; sl + 4 <= a.split; sl += 4) {
        float v[4][4];
#pragma unroll
        for (int q2 = 0; q2 < 4; ++q2) {
            const float *p = ws + (long)(sl + q2) * (BM * BN);
#pragma unroll
            for (int rr = 0; rr < 4; ++rr)
                v[q2][rr] = p[rr * 64];
        }
#pragma unroll
        for (int q2 = 0; q2 < 4; ++q2)
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) sum[rr] += v[q2][rr];
    }
    for (; sl < a.split; ++sl) {
        const float *p = ws + (long)sl * (BM * BN);
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) sum[rr] += p[rr * 64];
    }
    const int b = (int)((unsigned)n / (unsigned)a.P);
    const int px = (int)n - b * a.P;
    const conv_row_t row = conv_row(a, m);
    const long off = ((long)b * a.M + m) * a.P + px;
    float y[4];
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) y[rr] = conv_tail_one(sum[rr], row, conv_f2{a.slope_hi, a.slope_lo});
    if (px + 3 < a.P) { /* the four pixels lie in one image (then n + 3 < Ntotal too) */
        *(float4u *)(a.out + off) = (float4u){y[0], y[1], y[2], y[3]};
        if (a.yolo_entries) {
            const bool keep = conv_yolo_keeps(a, m);
            *(float4u *)(a.sum + off) = (float4u){conv_yolo_one(y[0], keep), conv_yolo_one(y[1], keep),
                                                  conv_yolo_one(y[2], keep), conv_yolo_one(y[3], keep)};
        } else if (a.sum) {
            const float4u r4 = *(const float4u *)(a.add + off);
            float4u s4;
            s4.x = conv_residual_one(a, y[0], r4.x);
            s4.y = conv_residual_one(a, y[1], r4.y);
            s4.z = conv_residual_one(a, y[2], r4.z);
            s4.w = conv_residual_one(a, y[3], r4.w);
            *(float4u *)(a.sum + off) = s4;
        }
    } else { /* image boundary or end of N inside the four: element by element */
        int pc = px;
        long offc = off;
        const long wrap = (long)(a.M - 1) * a.P; /* what the offset gains when the pixel index wraps */
        for (int rr = 0; rr < 4 && n + rr < a.Ntotal; ++rr) {
            while (pc >= a.P) {
                pc -= a.P;
                offc += wrap;
            }
            a.out[offc] = y[rr];
            if (a.yolo_entries)
                a.sum[offc] = conv_yolo_one(y[rr], conv_yolo_keeps(a, m));
            else if (a.sum)
                a.sum[offc] = conv_residual_one(a, y[rr], a.add[offc]);
            ++pc;
            ++offc;
        }
    }
}

/* BF16: 0 = fp32 operands; 1 = bf16 weights from their packed copy, fp32 activation tiles rounded
 * on the way into the MFMA (1x1 layers: the input is read once, straight from the fp32 tensor);
 * 2 = both operands bf16 in LDS, the activations gathered from a staged bf16 copy of the input
 * (3x3 layers, which read every input element nine times);
 * 3 = fp32 emulated on the bf16 matrix cores: every operand is the exact sum of three bf16 pieces
 * (x = hi + mid + lo, each the nearest-even rounding of what the previous ones left), the weights
 * pre-split into three packed copies, the activations split in registers from the fp32 LDS tile,
 * and a product is the six piece-products down to 2^-16 relative (hi*hi, hi*mid, mid*hi, hi*lo,
 * lo*hi, mid*mid; the three dropped ones are below 2^-24), accumulated in fp32. */
template <int BM, int BN, int WM, int WN, int MODE_V, int BF16 = 0>
__global__ __launch_bounds__(DN_THREADS, ((BM == 128 && BF16 != 3) ? 3 : 2)) void conv_mfma_kernel(mfma_args a)
{
    /* MODE_V = K order and kernel size, plus 100 for the variant that serves launches too small to
     * fill the chip (see the two forms of the fp32 loop below) */
    constexpr int MODE = MODE_V % 100;
    constexpr bool SPARSE_LAUNCH = MODE_V >= 100;
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int WAVES_N = BN / WN;
    static_assert((BM / WM) * (BN / WN) == 4, "four waves per workgroup");
    constexpr bool TAPB = MODE >= 10;             /* tap-blocked K order */
    constexpr int KS = TAPB ? MODE - 10 : MODE;    /* kernel size known at compile time (0 = runtime) */
    constexpr int TAPS = KS == 3 ? 9 : 1;

    /* Four separate LDS objects rather than two [2][...] arrays: the compiler makes every LDS read
     * wait (vmcnt) for direct-to-LDS loads it cannot prove disjoint from it, and it can only
     * prove that for distinct objects. */
    constexpr bool V3 = BF16 == 2;
    constexpr bool X3 = BF16 == 3;                 /* three-piece emulation: fp32-style pipeline */
    constexpr bool BFP = BF16 == 1 || BF16 == 2;    /* the deep-pipelined bf16 variants */
    static_assert(!V3 || (TAPB && KS == 3), "the staged-input variant serves the tap-blocked 3x3 layers");
    constexpr int A_FLOATS = X3 ? 3 * BM * DN_BK / 2 : BF16 ? BM * DN_BK / 2 : BM * DN_BK; /* bf16 rows are 32 bytes */
    constexpr int B_FLOATS = V3 ? BN * DN_BK / 2 : BN * DN_BK;
    __shared__ __attribute__((aligned(16))) float As0[V3 ? 4 : A_FLOATS], As1[V3 ? 4 : A_FLOATS];
    __shared__ __attribute__((aligned(16))) float Bs0[V3 ? 4 : B_FLOATS], Bs1[V3 ? 4 : B_FLOATS];
    /* the bf16 variants keep three chunks in flight: four stages */
    __shared__ __attribute__((aligned(16))) float As2[BF16 == 1 ? A_FLOATS : 4], As3[BF16 == 1 ? A_FLOATS : 4];
    __shared__ __attribute__((aligned(16))) float Bs2[BF16 == 1 ? B_FLOATS : 4], Bs3[BF16 == 1 ? B_FLOATS : 4];
    /* staged-input variant: one object per stage, [A | B], each at least the 8 KB a wave's
     * epilogue turn needs */
    constexpr int S_FLOATS = V3 ? A_FLOATS + B_FLOATS : 4;
    static_assert(!V3 || S_FLOATS >= 2048, "a stage doubles as one wave's epilogue buffer");
    __shared__ __attribute__((aligned(16))) float S0[S_FLOATS], S1[S_FLOATS], S2[S_FLOATS], S3[S_FLOATS];
#define S_BUF(b) ((b) == 0 ? S0 : (b) == 1 ? S1 : (b) == 2 ? S2 : S3)
    __shared__ conv_row_t rows_s[BM]; /* batch-norm constants of the tile's filters, for the epilogue */
#define A_BUF(b) (V3 ? S_BUF(b) : ((b) == 0 ? As0 : (b) == 1 ? As1 : (b) == 2 ? As2 : As3))
#define B_BUF(b) (V3 ? S_BUF(b) + A_FLOATS : ((b) == 0 ? Bs0 : (b) == 1 ? Bs1 : (b) == 2 ? Bs2 : Bs3))

    /* XCD-aware tile order: workgroup id -> (xcd, slot) -> linear tile with tile_m fastest. */
    const int bid = blockIdx.x;
    int lin, kc_begin = 0, kc_end = a.KCH, slice_id = -1;
    if (bid < 8 * a.per_xcd) {
        lin = (bid & 7) * a.per_xcd + (bid >> 3);
        if (lin >= a.whole_tiles) return;
    } else {
        slice_id = bid - 8 * a.per_xcd;
        const int t = slice_id / a.split, sl = slice_id - t * a.split;
        lin = a.whole_tiles + t;
        kc_begin = (int)((long)sl * a.KCH / a.split);
        kc_end = (int)((long)(sl + 1) * a.KCH / a.split);
    }
    const int band = lin / a.band_tiles, in_band = lin - band * a.band_tiles;
    const int tile_m = band * a.m_group + in_band % a.m_group;
    const int tile_n = in_band / a.m_group;
    const int m0 = tile_m * BM;
    const long n0 = (long)tile_n * BN;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave / WAVES_N) * WM;
    const int wn0 = (wave % WAVES_N) * WN;

    /* ---- global -> LDS without passing through registers ------------------------------------
     * A buffer load with the LDS modifier writes lane i's dword (or 16 bytes) to
     * lds_base + i*4 (i*16); lanes whose offset is out of range write zeros.  The layouts are
     * chosen so that those wave-contiguous images are exactly what the MFMA operand reads want:
     *   LDS   A: [slot q = 0..3][row m][4 floats],  B: [slot q][column n][4 floats]  (k = 4q + j)
     *   A wave-load: 64 rows of one slot, 16 bytes per lane - the packed weights are stored
     *                [chunk][slot][Mpad][4] so this is one contiguous kilobyte;
     *   B wave-load: 16 consecutive columns x the 4 k of one slot, lane = 4*column + j.
     * No ds_write, no staging registers; completion is tracked by vmcnt. */
    constexpr int A_WAVE_LOADS = BM * 4 / 64;            /* wave-loads of A per chunk (8, 4 or 2) */
    constexpr int A_PER_WAVE = (A_WAVE_LOADS + 3) / 4;   /* 2, 1, 1 */
    constexpr int NG = BN / 16;                          /* 16-column groups per tile */
    constexpr int NG_PER_WAVE = NG / 4;                  /* 2 (BN=128) or 4 (BN=256) */
    const int nl = lane >> 2;                            /* column inside a 16-group */
    const int kk = lane & 3;                             /* k inside a slot */
    const int HW = a.H * a.W;

    const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(BF16 ? a.wp16 : (const void *)a.wp), 0, (int)(BF16 ? a.wp16_records : a.wp_records), 0x00020000);
    const int bias = (TAPB && KS == 3) ? a.W + 1 : 0;
    const __amdgpu_buffer_rsrc_t in_rsrc =
        V3 ? __builtin_amdgcn_make_buffer_rsrc((void *)((const char *)a.in16 - (long)bias * 16), 0, (int)a.in16_records,
                                               0x00020000)
           : __builtin_amdgcn_make_buffer_rsrc((void *)(a.in - bias), 0, (int)a.in_records, 0x00020000);

    /* per column group handled by this wave: the lane's pixel */
    unsigned voff_px[NG_PER_WAVE]; /* byte offset of (image, channel kk [tap-blocked] or 0, oy*s, ox*s) */
    unsigned vmask[NG_PER_WAVE];   /* tap-blocked: bit t set when tap t lies inside the image */
    int iy0[NG_PER_WAVE], ix0[NG_PER_WAVE]; /* reference order: top-left input pixel of the window;
                                             * a column beyond N gets iy0 far outside the image */
    /* staged-input variant: the input is [image][C/8][H*W] rows of eight bf16 channels, so a lane
     * fetches a column's eight k of one half with one 16-byte load: a wave-load is 64 consecutive
     * columns of one k half, and this wave serves half `lkh`, 64-column blocks lblk0 .. */
    constexpr int NBW = V3 ? BN / 128 : 1;       /* 64-column blocks per wave */
    const int lkh = wave >> 1, lblk0 = (wave & 1) * NBW;
    unsigned c_voff[NBW], c_mask[NBW];
    if constexpr (V3) {
#pragma unroll
        for (int g = 0; g < NBW; ++g) {
            const long ncol = n0 + (lblk0 + g) * 64 + lane;
            const bool col_ok = ncol < a.Ntotal;
            const unsigned nn = col_ok ? (unsigned)ncol : 0u;
            const int b = (int)(nn / (unsigned)a.P);
            const int p = (int)nn - b * a.P;
            const int oy = (int)((unsigned)p / (unsigned)a.OW);
            const int ox = p - oy * a.OW;
            const int y0 = oy * a.stride - 1, x0 = ox * a.stride - 1; /* pad == 1 */
            c_voff[g] = (unsigned)((((long)b * (a.C >> 3) + lkh) * HW + (long)(oy * a.stride) * a.W + ox * a.stride) * 16);
            c_mask[g] = 0;
            if (col_ok) {
#pragma unroll
                for (int t = 0; t < 9; ++t)
                    if ((unsigned)(y0 + t / 3) < (unsigned)a.H && (unsigned)(x0 + t % 3) < (unsigned)a.W) c_mask[g] |= 1u << t;
            }
        }
    }
#pragma unroll
    for (int g = 0; g < NG_PER_WAVE; ++g) {
        const long ncol = n0 + (wave * NG_PER_WAVE + g) * 16 + nl;
        const bool col_ok = ncol < a.Ntotal;
        const unsigned nn = col_ok ? (unsigned)ncol : 0u; /* Ntotal < 2^31 on this path */
        const int b = (int)(nn / (unsigned)a.P);
        const int p = (int)nn - b * a.P;
        const int oy = (int)((unsigned)p / (unsigned)a.OW);
        const int ox = p - oy * a.OW;
        iy0[g] = col_ok ? oy * a.stride - a.pad : -0x1000000;
        ix0[g] = ox * a.stride - a.pad;
        const long img = (long)b * a.C * HW;
        vmask[g] = 0;
        if (TAPB) {
            voff_px[g] = (unsigned)((img + (long)kk * HW + (long)(oy * a.stride) * a.W + ox * a.stride) * 4);
            if (col_ok) {
#pragma unroll
                for (int t = 0; t < TAPS; ++t) {
                    const int ky = t / 3, kx = t % 3;
                    if (KS == 1 || ((unsigned)(iy0[g] + ky) < (unsigned)a.H && (unsigned)(ix0[g] + kx) < (unsigned)a.W))
                        vmask[g] |= 1u << t;
                }
            }
        } else {
            /* (image, channel 0, window origin); the origin may lie above/left of the image, the
             * sum with a valid tap's offset never does */
            voff_px[g] = (unsigned)((img + (long)(oy * a.stride - a.pad) * a.W + (ox * a.stride - a.pad)) * 4);
        }
    }
    /* tap-blocked loop state of the chunk being fetched (wave-uniform) */
    int ld_cb = kc_begin / TAPS + (a.grouped ? tile_m * 2 : 0), ld_tap = kc_begin - (kc_begin / TAPS) * TAPS;

    typedef __attribute__((address_space(3))) void *lds_ptr;

    /* `live` = false: the request is only there to keep a schedule region free of branches (the last
     * step of a loop form that always requests "the next chunk").  Its weights are chunk kc's again
     * (in range by construction); its input lanes all carry the out-of-range offset, so they write
     * zeros to LDS and read no memory.  (The tap-blocked input address of such a request would be one
     * chunk past the layer's channels; for the last image that lies past the tensor, where only the
     * buffer's range check - which on this part covers the scalar offset too - stands between the
     * request and the memory behind the tensor.  A request that is not live does not lean on it.) */
    auto load_chunk = [&](int kc, int buf, bool live = true) {
        /* A */
        if constexpr (BF16) {
            /* bf16 copy: [chunk][k half][Mpad16 rows][8 bf16]; LDS image [k half][BM][16 bytes].
             * A wave-load moves 64 consecutive 16-byte rows of one k half (both halves of the 32
             * rows when BM == 32). */
            constexpr int WL = BM / 32;                  /* wave-loads per chunk: 8, 4, 2, 1 */
            constexpr int PER_WAVE = (WL + 3) / 4;
            constexpr int PLANES = X3 ? 3 : 1;           /* hi (, mid, lo) copies, a.plane16 bytes apart */
#pragma unroll
            for (int pl = 0; pl < PLANES; ++pl) {
#pragma unroll
                for (int i = 0; i < PER_WAVE; ++i) {
                    const int wl = wave * PER_WAVE + i;
                    if (WL >= 4 || wl < WL) {
                        if (BM >= 64) {
                            constexpr int RB = BM / 64;
                            const int h = wl / RB, rb = wl - h * RB;
                            const unsigned soff =
                                (unsigned)((((long)kc * 2 + h) * a.Mpad16 + m0 + rb * 64) * 16) + pl * a.plane16;
                            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                                w_rsrc, (lds_ptr)&A_BUF(buf)[pl * BM * 8 + (h * BM + rb * 64) * 4], 16, lane * 16, soff, 0, 0);
                        } else {
                            const unsigned voff = (unsigned)((((long)(lane >> 5) * a.Mpad16) + (lane & 31)) * 16);
                            const unsigned soff = (a.grouped ? (unsigned)(((long)(tile_m * a.KCH + kc) * 2 * 32) * 16)
                                                             : (unsigned)(((long)kc * 2 * a.Mpad16 + m0) * 16)) +
                                                  pl * a.plane16;
                            __builtin_amdgcn_raw_ptr_buffer_load_lds(w_rsrc, (lds_ptr)&A_BUF(buf)[pl * BM * 8], 16, voff, soff,
                                                                     0, 0);
                        }
                    }
                }
            }
        } else {
#pragma unroll
        for (int i = 0; i < A_PER_WAVE; ++i) {
            const int wl = wave * A_PER_WAVE + i;        /* wave-load index: slot q, 64-row block rb */
            if (A_WAVE_LOADS >= 4 || wl < A_WAVE_LOADS) {
                constexpr int RB = BM / 64 > 0 ? BM / 64 : 1; /* 64-row blocks per slot (BM >= 64) */
                const int q = BM >= 64 ? wl / RB : wl / 1;
                const int rb = BM >= 64 ? wl - q * RB : 0;
                if (BM >= 64) {
                    const unsigned soff = (unsigned)((((long)kc * 4 + q) * a.Mpad + m0 + rb * 64) * 16);
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(w_rsrc, (lds_ptr)&A_BUF(buf)[(q * BM + rb * 64) * 4], 16,
                                                             lane * 16, soff, 0, 0);
                } else {
                    /* BM == 32: one wave-load covers two slots of 32 rows each */
                    const int q2 = wl * 2 + (lane >> 5);
                    const unsigned voff = (unsigned)((((long)q2 * a.Mpad) + (lane & 31)) * 16);
                    /* grouped: Mpad == 32 and the tile's chunks follow each other */
                    const unsigned soff = a.grouped ? (unsigned)(((long)(tile_m * a.KCH + kc) * 4 * 32) * 16)
                                                    : (unsigned)(((long)kc * 4 * a.Mpad + m0) * 16);
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(w_rsrc, (lds_ptr)&A_BUF(buf)[(wl * 2 * BM) * 4], 16, voff,
                                                             soff, 0, 0);
                }
            }
        }
        }
        /* B */
        if constexpr (V3) {
            const int ky = (ld_tap * 11) >> 5, kx = ld_tap - 3 * ((ld_tap * 11) >> 5); /* tap/3, tap%3 */
            const int shift = (ky - 1) * a.W + (kx - 1);
            const unsigned soff0 = (unsigned)(((long)2 * ld_cb * HW + shift + bias) * 16); /* wave-uniform */
            const int tap_bit = live ? ld_tap : 31; /* bit 31 of a tap mask is never set */
#pragma unroll
            for (int g = 0; g < NBW; ++g) {
                const unsigned voff = ((c_mask[g] >> tap_bit) & 1u) ? c_voff[g] : 0xFFFFFFF0u;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(in_rsrc, (lds_ptr)&B_BUF(buf)[(lkh * BN + (lblk0 + g) * 64) * 4], 16,
                                                         voff, soff0, 0, 0);
            }
            if (++ld_tap == TAPS) {
                ld_tap = 0;
                ++ld_cb;
            }
        } else if (TAPB) {
            const int ky = (ld_tap * 11) >> 5, kx = ld_tap - 3 * ((ld_tap * 11) >> 5); /* tap/3, tap%3 */
            const int shift = KS == 1 ? 0 : (ky - 1) * a.W + (kx - 1);       /* pad == 1 for 3x3 */
            const unsigned soff0 = (unsigned)((ld_cb * 16 * HW + shift + bias) * 4); /* wave-uniform */
            const int tap_bit = live ? ld_tap : 31; /* bit 31 of a tap mask is never set */
#pragma unroll
            for (int g = 0; g < NG_PER_WAVE; ++g) {
                const unsigned voff = ((vmask[g] >> tap_bit) & 1u) ? voff_px[g] : 0xFFFFFFFCu;
                const int ng = wave * NG_PER_WAVE + g;
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(in_rsrc, (lds_ptr)&B_BUF(buf)[(q * BN + ng * 16) * 4], 4,
                                                             voff, soff0 + (unsigned)(q * 4 * HW * 4), 0, 0);
            }
            if (++ld_tap == TAPS) {
                ld_tap = 0;
                ++ld_cb;
            }
        } else {
            /* reference K order: every lane splits its own k (4 per chunk, one per slot) */
            int koff[4];
            int kyx[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int k = kc * DN_BK + q * 4 + kk;
                int ci, ky, kx;
                split_k<KS>(k, a.size, ci, ky, kx);
                koff[q] = (ci * HW + ky * a.W + kx) * 4;
                kyx[q] = k < a.K ? (ky << 16) | kx : 0x7fff0000; /* k beyond K: fails the row test */
            }
#pragma unroll
            for (int g = 0; g < NG_PER_WAVE; ++g) {
                const int ng = wave * NG_PER_WAVE + g;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int ky = kyx[q] >> 16, kx = kyx[q] & 0xffff;
                    const bool ok = live & ((unsigned)(iy0[g] + ky) < (unsigned)a.H) & ((unsigned)(ix0[g] + kx) < (unsigned)a.W);
                    const unsigned voff = ok ? voff_px[g] + (unsigned)koff[q] : 0xFFFFFFFCu;
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(in_rsrc, (lds_ptr)&B_BUF(buf)[(q * BN + ng * 16) * 4], 4,
                                                             voff, 0, 0, 0);
                }
            }
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

    /* loads one wave issues per chunk, for the s_waitcnt immediates of the bf16 pipeline (the A
     * loads are left out where not every wave issues them: those waves wait for one load more
     * than they must) */
    constexpr int LPC = (BFP && BM >= 128 ? BM / 128 : 0) + (V3 ? NBW : 4 * NG_PER_WAVE);
    /* s_waitcnt on vmcnt alone: simm16 = vmcnt[3:0] | expcnt(7) << 4 | lgkmcnt(15) << 8 | vmcnt[5:4] << 14 */
#define DN_WAIT_VM(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (7 << 4) | (15 << 8) | (((n) >> 4) << 14))
    static_assert(2 * LPC < 64, "vmcnt is a 6-bit counter");

    float4 av[2][TM], bv[BF16 == 1 ? 2 : 1][2][TN]; /* MFMA operands of a chunk: [k half][32-row block] */
    bf16x8 a8[2][BFP ? TM : 1];              /* bf16 modes: a row's eight k of this lane's half, two register sets */
    bf16x8 a3[3][X3 ? TM : 1];               /* three-piece mode: hi, mid, lo of the same */
    bf16x8 b8s[2][V3 ? TN : 1];              /* staged input: a column's eight k likewise */

    auto read_operands = [&](int buf, int r) {
#pragma unroll
        for (int hb = 0; hb < 2; ++hb) {
            if constexpr (!BF16) {
#pragma unroll
                for (int i = 0; i < TM; ++i)
                    av[hb][i] = *(const float4 *)&A_BUF(buf)[((hb * 2 + kh) * BM + wm0 + i * 32 + li) * 4];
            }
            if constexpr (!V3) {
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    /* which two slots hold this lane's eight k: (kh, 2 + kh) as the fp32 layout pairs them,
                     * or (2kh, 2kh + 1) where the bf16 copy of a 3x3 layer is packed eight channels per half */
                    bv[BF16 == 1 ? r : 0][hb][j] =
                        *(const float4 *)&B_BUF(buf)[(((X3 && KS == 3) ? 2 * kh + hb : hb * 2 + kh) * BN + wn0 + j * 32 + li) * 4];
            }
        }
        if constexpr (BFP) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
                a8[r][i] = *(const bf16x8 *)&A_BUF(buf)[(kh * BM + wm0 + i * 32 + li) * 4];
        }
        if constexpr (X3) {
#pragma unroll
            for (int pl = 0; pl < 3; ++pl)
#pragma unroll
                for (int i = 0; i < TM; ++i)
                    a3[pl][i] = *(const bf16x8 *)&A_BUF(buf)[pl * BM * 8 + (kh * BM + wm0 + i * 32 + li) * 4];
        }
        if constexpr (V3) {
#pragma unroll
            for (int j = 0; j < TN; ++j)
                b8s[r][j] = *(const bf16x8 *)&B_BUF(buf)[(kh * BN + wn0 + j * 32 + li) * 4];
        }
    };

    if constexpr (BFP) {
        /* chunks 0..2 requested; chunks 0 and 1 must have landed before the first step */
        const int nch = kc_end - kc_begin;
        load_chunk(kc_begin, 0);
        if (nch > 1) load_chunk(kc_begin + 1, 1);
        if (nch > 2) load_chunk(kc_begin + 2, 2);
        if (nch > 2)
            DN_WAIT_VM(LPC);
        else
            __builtin_amdgcn_s_waitcnt(0);
        __builtin_amdgcn_s_barrier();
        read_operands(0, 0);
    } else {
        load_chunk(kc_begin, 0);
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
    }

    auto mfma_half = [&](int hb) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const float ae = s == 0 ? av[hb][i].x : s == 1 ? av[hb][i].y : s == 2 ? av[hb][i].z : av[hb][i].w;
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    const float4 b4 = bv[0][hb][j];
                    const float be = s == 0 ? b4.x : s == 1 ? b4.y : s == 2 ? b4.z : b4.w;
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(be, ae, acc[i][j], 0, 0, 0);
                }
            }
        }
    };

    /* Reduced-precision variants: the weights come from their bf16 copy, whose rows hold the eight
     * k of a lane half in the order the activations give them.  Variant 1 keeps the activations
     * as fp32 tiles in LDS and rounds them to bf16 (nearest even) on the way into the MFMA;
     * variant 2 reads them already rounded from the staged copy.  One v_mfma_f32_32x32x16_bf16
     * contracts all 16 k of the chunk; products and sums stay fp32, so does everything after the
     * accumulators. */
    auto mfma_chunk = [&](int r) {
        if constexpr (X3) {
            /* x = hi + mid + lo: hi = bf16(x), mid = bf16(x - hi), lo = bf16(x - hi - mid); both
             * subtractions are exact in fp32.  Small terms first. */
            bf16x8 bh[TN], bm[TN], bl[TN];
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const float4 q0 = bv[0][0][j], q1 = bv[0][1][j];
                const f32x8 f = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
                bh[j] = __builtin_convertvector(f, bf16x8);
                const f32x8 r1 = f - __builtin_convertvector(bh[j], f32x8);
                bm[j] = __builtin_convertvector(r1, bf16x8);
                const f32x8 r2 = r1 - __builtin_convertvector(bm[j], f32x8);
                bl[j] = __builtin_convertvector(r2, bf16x8);
            }
            /* term by term over all accumulators, so that consecutive MFMAs are independent */
#define DN_X3_TERM(BOP, APL)                                                                        \
    _Pragma("unroll") for (int i = 0; i < TM; ++i) _Pragma("unroll") for (int j = 0; j < TN; ++j)  \
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(BOP[j], a3[APL][i], acc[i][j], 0, 0, 0)
            DN_X3_TERM(bl, 0); /* lo  * hi  */
            DN_X3_TERM(bh, 2); /* hi  * lo  */
            DN_X3_TERM(bm, 1); /* mid * mid */
            DN_X3_TERM(bm, 0); /* mid * hi  */
            DN_X3_TERM(bh, 1); /* hi  * mid */
            DN_X3_TERM(bh, 0); /* hi  * hi  */
#undef DN_X3_TERM
        } else if constexpr (BF16) {
            bf16x8 b8[TN];
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if constexpr (V3) {
                    b8[j] = b8s[r][j];
                } else {
                    const float4 lo = bv[BF16 == 1 ? r : 0][0][j], hi = bv[BF16 == 1 ? r : 0][1][j];
                    const f32x8 f = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
                    b8[j] = __builtin_convertvector(f, bf16x8);
                }
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b8[j], a8[r][i], acc[i][j], 0, 0, 0);
        } else {
            mfma_half(0);
            mfma_half(1);
        }
    };

    /* One pipeline step, in program order (pinned by scheduling barriers):
     *   1. LDS operand reads of chunk kc are issued
     *   2. while they are under way, direct-to-LDS loads of chunk kc+1 into the other buffer
     *      (nobody reads it: every wave passed the previous barrier only after its MFMAs had
     *      consumed that buffer); the two swap places for the tiles with 256 columns
     *   3. the MFMAs of chunk kc
     *   4. wait for this wave's loads (vmcnt), barrier: chunk kc+1 is now visible to all waves */
    /* loads a wave issues per chunk in the fp32 kernels, and the MFMAs of the chunk that go in front of each */
    constexpr int LPC_F = A_PER_WAVE + 4 * NG_PER_WAVE;
    constexpr int MFMA_PER_LOAD = (8 * TM * TN) / (LPC_F + 1) > 0 ? (8 * TM * TN) / (LPC_F + 1) : 1;
    auto step = [&](int kc_next, int buf) {
        if constexpr (!BF16) {
            /* fp32: the next chunk's loads are issued between this chunk's MFMAs */
            read_operands(buf, 0);
            __builtin_amdgcn_sched_barrier(0);
            load_chunk(kc_next, buf ^ 1);
            mfma_chunk(0);
#pragma unroll
            for (int g = 0; g < LPC_F; ++g) {
                __builtin_amdgcn_sched_group_barrier(0x008, MFMA_PER_LOAD, 0);
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
            return;
        }
        /* the 128-row tiles gain 1-5% from having their reads under way while the loads are issued;
         * the 256-column tiles, with twice the loads per wave, lose 7% and keep loads first */
        if constexpr (BM >= 128) {
            read_operands(buf, 0);
            __builtin_amdgcn_sched_barrier(0);
            load_chunk(kc_next, buf ^ 1);
        } else {
            load_chunk(kc_next, buf ^ 1);
            __builtin_amdgcn_sched_barrier(0);
            read_operands(buf, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        mfma_chunk(0);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
    };
    /* The last chunk requests nothing.  Invariant of every way out of the chunk loop: no wave leaves it
     * with a direct-to-LDS load in flight (vmcnt = 0) - every step above ends with s_waitcnt(0) in
     * front of its barrier, and `last` issues no load - so neither the epilogue's reuse of the LDS
     * buffers nor the end of a K-slice workgroup (which gives its LDS back) can meet a pending write. */
    auto last = [&](int buf) {
        read_operands(buf, 0);
        mfma_chunk(0);
    };

    if constexpr (BFP) {
        /* Four LDS stages and two register sets.  A bf16 chunk is 8 (or 4, 2) MFMAs, far shorter
         * than a trip to memory or even to LDS, so a step overlaps three things: the LDS reads of
         * chunk kc+1 into the other register set, the request for chunk kc+3, and the MFMAs of
         * chunk kc from registers read one step earlier.  On entry chunks up to kc+1 are in LDS
         * and visible, chunk kc+2 is in flight; the step ends when kc+2 has landed for every wave
         * (vmcnt counts this wave's loads, which complete in order; the barrier publishes them).
         * The stage requested into is the one of chunk kc-1, last read two steps ago.
         * __syncthreads() would drain every load (its fences wait for vmcnt(0) because
         * direct-to-LDS loads count as LDS writes), so the barrier is the bare instruction. */
        auto bstep = [&](int kcur, int buf, int r) {
            const int rem = kc_end - 1 - kcur; /* chunks after this one (wave-uniform) */
            if (rem >= 1) read_operands((buf + 1) & 3, r ^ 1);
            __builtin_amdgcn_sched_barrier(0);
            if (rem >= 3) load_chunk(kcur + 3, (buf + 3) & 3);
            __builtin_amdgcn_sched_barrier(0);
            mfma_chunk(r);
            __builtin_amdgcn_sched_barrier(0);
            if (rem >= 3)
                DN_WAIT_VM(LPC);
            else
                DN_WAIT_VM(0);
            if (rem >= 2) __builtin_amdgcn_s_barrier();
        };
        for (int kc = kc_begin; kc < kc_end; kc += 4) {
            bstep(kc, 0, 0);
            if (kc + 1 < kc_end) bstep(kc + 1, 1, 1);
            if (kc + 2 < kc_end) bstep(kc + 2, 2, 0);
            if (kc + 3 < kc_end) bstep(kc + 3, 3, 1);
        }
    } else if constexpr (!BF16 && !X3 && BM >= 128 && !SPARSE_LAUNCH) {
        /* fp32, 128-row tiles in launches that fill the chip: the step with the number of chunks still
         * to come as a run-time scalar instead of a peeled last chunk.  The compiler then keeps 71 (128x64)
         * and 115 (128x128) vector registers live instead of 102 and 168, so a CU holds five and four
         * workgroups instead of four and three, and its matrix pipe idles less while one of them is in
         * its prologue or epilogue: 2-3% less time per 3x3 layer at batch 64, 12% on 512->1024 at 13x13
         * with the 128x64 tile.  A workgroup alone on its CU (batch 1) is 1-4% faster with the peeled
         * form below, which the +100 variants keep; so are the 64- and 32-row tiles (no more workgroups
         * fit: 64x64 already holds eight). */
        auto fstep = [&](int kcur, int buf) {
            const int rem = kc_end - 1 - kcur; /* chunks after this one (wave-uniform) */
            read_operands(buf, 0);
            __builtin_amdgcn_sched_barrier(0);
            /* the next chunk's loads go between this chunk's MFMAs (the last step requests its own
             * chunk again: no branch inside the schedule region) */
            load_chunk(rem >= 1 ? kcur + 1 : kcur, buf ^ 1, rem >= 1);
            mfma_chunk(0);
#pragma unroll
            for (int g = 0; g < LPC_F; ++g) {
                __builtin_amdgcn_sched_group_barrier(0x008, MFMA_PER_LOAD, 0);
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            /* also after the last chunk: its repeated request must have landed before the workgroup
             * reuses its LDS in the epilogue or, as a K-slice, ends and gives it back */
            __builtin_amdgcn_s_waitcnt(0);
            if (rem >= 1) __syncthreads();
        };
        for (int kc = kc_begin; kc < kc_end; kc += 2) {
            fstep(kc, 0);
            if (kc + 1 < kc_end) fstep(kc + 1, 1);
        }
    } else {
    int kc = kc_begin;
    /* two chunks per trip so the LDS buffer index is a compile-time constant in each half */
    for (; kc + 2 < kc_end; kc += 2) {
        step(kc + 1, 0);
        step(kc + 2, 1);
    }
    if (kc + 1 < kc_end) { /* even count: one more full step, then the last chunk from buffer 1 */
        step(kc + 1, 0);
        last(1);
    } else {
        last(0);
    }

    }

    /* here vmcnt = 0 on every path (see `last` and `fstep`) */
    if (slice_id >= 0) {
        /* K-slice: park the raw accumulators, lane-major so every store is a full 256-byte row */
        float *ws = a.partial + (long)slice_id * (BM * BN);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    ws[((wave * TM * TN + i * TN + j) * 16 + r) * 64 + lane] = acc[i][j][r];
    } else {
        /* The per-filter constants cost a double-precision square root and division each: one lane
         * per filter of the tile computes them once (every wave would otherwise repeat them for
         * each of its 32-row blocks, on the vector ALU the fp32 MFMAs of the other waves need). */
        if (tid < BM) rows_s[tid] = conv_row(a, m0 + tid < a.M ? m0 + tid : a.M - 1);
        __syncthreads(); /* every wave has read its last operands: the LDS buffers are free */
        float *E = V3 ? S_BUF(wave)
                   : (BM >= 128 || BN == 64) ? (BFP ? (wave == 0 ? Bs2 : wave == 1 ? Bs3 : wave == 2 ? Bs0 : Bs1)
                                                    : (wave == 0 ? As0 : wave == 1 ? As1 : wave == 2 ? Bs0 : Bs1))
                                             : (wave < 2 ? Bs0 : Bs1) + (wave & 1) * 2048;
        static_assert(BN != 64 || (A_FLOATS >= 32 * 32 * TN && B_FLOATS >= 32 * 32 * TN),
                      "each operand buffer holds one wave's turn of 32 filters x 32*TN pixels");
        conv_epilogue<TM, TN>(a, acc, E, rows_s, m0, n0, wm0, wn0, lane);
    }
}

/* The reduction is a launch of its own, of many small workgroups: a handful of tail tiles must
 * still spread over the whole chip.  (Letting the slices of a tile wait for each other and sum
 * themselves inside the main launch was built and measured, with the slices placed on one XCD
 * and talking through its L2: correct, and no faster - every hand-over between workgroups costs
 * a round trip of 0.5-1 microsecond even inside an XCD, and storing, announcing, polling, loading
 * and leaving add up to what the second launch costs.) */
template <int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(DN_THREADS) void conv_reduce_kernel(mfma_args a)
{
    constexpr int GROUPS_PER_TILE = BM * BN / 4 / DN_THREADS; /* workgroups per tile */
    const int t = blockIdx.x / GROUPS_PER_TILE;
    const int u = (blockIdx.x - t * GROUPS_PER_TILE) * DN_THREADS + threadIdx.x;
    conv_reduce_unit<BM, BN, WM, WN>(a, t, u);
}

/* ---- first layers: 3 input channels, 3x3, stride 1, pad 1 --------------------------------- */
/* With K = 27 the general kernel spends its time on the gather (one 4-byte load per column and k,
 * each with its own index split) and on per-tile index arithmetic, not on its two chunks of MFMAs.
 * Here a workgroup owns 256 consecutive output pixels of one image and every filter: it copies
 * the input rows those pixels touch into LDS once (16 bytes per lane, zero columns left and right
 * and zero rows above and below the image, so no tap needs a border test), keeps the weights in
 * registers (a lane holds its filter's 14 k of the MFMA's k pairs), and feeds the MFMAs from LDS
 * with one 4-byte read per pixel and k: address = pixel base + a per-k offset.  K order is the
 * reference's (channel, ky, kx), padded from 27 to 28.  Accumulators are laid out as in
 * conv_mfma_kernel (pixel rows, filter columns), so the epilogue is shared.  The layer is bound by
 * writing its output (32 filters x 416 x 416: 22 MB per image for 0.6 MB read). */
#define DN_PATCH_FLOATS 8192     /* at most 32 KB for the input rows of a tile */
#define DN_PATCH_MIN_FLOATS 4096 /* 16 KB: the buffer also turns 16 filters x 256 pixels for the store */
extern __shared__ __attribute__((aligned(16))) float conv_patch_lds[];
template <int TM, int C>
__global__ __launch_bounds__(DN_THREADS, 4) void conv_patch_kernel(mfma_args a)
{
    constexpr int K = 9 * C, NS = (K + 1) / 2; /* MFMA k pairs */
    typedef __attribute__((address_space(3))) void *lds_ptr;
    float *buf = conv_patch_lds; /* sized by the launch: the tile's input rows (what the geometry needs, so
                                  * that as many tiles as possible are in flight on a CU: their trips to
                                  * memory, not their arithmetic, are what takes the time) */
    __shared__ __attribute__((aligned(16))) float wsm[TM * 32 * K]; /* the weights, as they lie in memory */
    __shared__ conv_row_t rows_s[TM * 32];
    const int tid = threadIdx.x, lane = tid & 63, li = lane & 31, kh = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int W = a.W, H = a.H, P = a.P;
    const int tiles_per_image = P / 256; /* the host checks P % 256 == 0 */
    /* Workgroup ids go round the eight XCDs, each with an L2 of its own, and neighbouring tiles
     * share input rows (a 256-pixel tile reads three or four rows to produce part of one): XCD x
     * takes the x-th eighth of the tile order, so that neighbours meet in one L2 instead of each
     * fetching those rows into its own. */
    const int ntiles = gridDim.x, xq = ntiles >> 3, xr = ntiles & 7, xcd = blockIdx.x & 7;
    const int tile = xcd * xq + (xcd < xr ? xcd : xr) + (blockIdx.x >> 3);
    const int b = tile / tiles_per_image;
    const int p0 = (tile - b * tiles_per_image) * 256;
    const int y0 = p0 / W, y1 = (p0 + 255) / W;
    const int nrows = y1 - y0 + 3, RS = W + 8; /* a row: four zeros, the W pixels, four zeros */

    /* Input rows y0-1 .. y1+1 of every channel, copied by loads that write straight to LDS, 16
     * bytes per lane: the patch is one flat array of C * nrows * RS / 4 quads cut into wave-loads
     * of 64 consecutive quads, dealt round-robin to the four waves; lane i of a wave-load owns quad
     * 64 * segment + i = (channel-row cr, quad qx of the row), walked without divisions.  W is a
     * multiple of 4, so a quad is either four pixels of one row or padding; quads of padding, of
     * rows outside the image and past the end of the patch carry an offset beyond the buffer's
     * range and arrive as zeros. */
    const __amdgpu_buffer_rsrc_t in_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(a.in + (long)b * C * H * W), 0, C * H * W * 4, 0x00020000);
    const int RQ = RS >> 2, total = C * nrows * RQ; /* quads per row, quads in all */
    {
        int e = wave * 64 + lane;
        int cr = e / RQ, qx = e - cr * RQ;       /* one division per lane */
        int ci = cr / nrows, r = cr - ci * nrows;
        for (int seg = wave; seg * 64 < total; seg += 4) {
            const int iy = y0 - 1 + r;
            const bool ok = e < total && (unsigned)iy < (unsigned)H && qx >= 1 && qx < RQ - 1;
            const unsigned voff = ok ? (unsigned)(((ci * H + iy) * W + 4 * (qx - 1)) * 4) : 0xFFFFFFF0u;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(in_rsrc, (lds_ptr)&buf[seg * 256], 16, voff, 0, 0, 0);
            e += 256;
            qx += 256;
            while (qx >= RQ) {
                qx -= RQ;
                if (++r == nrows) {
                    r = 0;
                    ++ci;
                }
            }
        }
    }
    /* the weights of all filters, coalesced, then each lane picks its own: filter 32i + li,
     * k = 2s + kh in (channel, ky, kx) order (rows are 27 floats apart: no bank conflicts) */
    for (int i = tid; i < TM * 32 * K; i += DN_THREADS) wsm[i] = i < a.M * K ? a.wp[i] : 0.f;
    if (tid < TM * 32) rows_s[tid] = conv_row(a, tid < a.M ? tid : a.M - 1);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();

    float aw[TM][NS];
    int koff[NS]; /* LDS offset of k relative to the pixel's base (row y - y0, column x) */
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        const int k = 2 * s + kh;
        const int ci = k / 9, r9 = k - 9 * ci, ky = r9 / 3, kx = r9 - 3 * ky;
        koff[s] = k < K ? (ci * nrows + ky) * RS + kx + 3 : 0; /* pixel x sits in column x + 4 */
#pragma unroll
        for (int i = 0; i < TM; ++i) aw[i][s] = k < K ? wsm[(i * 32 + li) * K + k] : 0.f;
    }

    f32x16 acc[TM][2];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    int base[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int p = p0 + wave * 64 + j * 32 + li;
        const int y = (int)((unsigned)p / (unsigned)W);
        base[j] = (y - y0) * RS + (p - y * W);
    }
#pragma unroll
    for (int s = 0; s < NS; ++s) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const float bv = buf[base[j] + koff[s]];
#pragma unroll
            for (int i = 0; i < TM; ++i) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv, aw[i][s], acc[i][j], 0, 0, 0);
        }
    }
    /* Tail and store.  The output is what bounds this layer, and memory takes whole kilobytes
     * better than the 256-byte pieces a wave's own 64 pixels make per filter: the four waves pool
     * their finished values in LDS, 16 filters x 256 pixels at a time (16-byte quads XOR-swizzled
     * by the filter), and each wave then stores four filter rows, one contiguous kilobyte per
     * instruction. */
    const long out_base = ((long)b * a.M) * P + p0;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const conv_row_t row = rows_s[i * 32 + li];
        /* the tail arithmetic with every lane at work; only the turn through LDS below goes by halves */
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[i][j][r] = conv_tail_one(acc[i][j][r], row, conv_f2{a.slope_hi, a.slope_lo});
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            __syncthreads(); /* the buffer is free: pixels read (first pass), rows stored (later ones) */
            if ((li >> 4) == hf) {
                const int f16 = li & 15;
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int rg = 0; rg < 4; ++rg) {
                        float4 o;
                        o.x = acc[i][j][rg * 4 + 0];
                        o.y = acc[i][j][rg * 4 + 1];
                        o.z = acc[i][j][rg * 4 + 2];
                        o.w = acc[i][j][rg * 4 + 3];
                        const int q = wave * 16 + j * 8 + 2 * rg + kh; /* quad of four pixels within the tile */
                        *(float4 *)&buf[f16 * 256 + ((q ^ f16) << 2)] = o;
                    }
            }
            __syncthreads();
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int f16 = wave * 4 + t, m = i * 32 + hf * 16 + f16;
                const float4 o = *(const float4 *)&buf[f16 * 256 + ((lane ^ f16) << 2)];
                if (m < a.M) *(float4u *)(a.out + out_base + (long)m * P + 4 * lane) = (float4u){o.x, o.y, o.z, o.w};
            }
        }
    }
}

/* Floats of LDS a tile's input rows take (0: conv_patch_kernel does not serve the layer). */
static long conv_patch_floats(int c, int h, int w, int n, int groups, int size, int stride, int pad)
{
    if (groups != 1 || c != 3 || size != 3 || stride != 1 || pad != 1 || n > 64) return 0;
    const long P = (long)h * w;
    if (P % 256 || w % 4) return 0; /* whole tiles per image; rows are copied 16 bytes at a time */
    if ((long)3 * h * w * 4 >= (1L << 31)) return 0;
    const long rows = 255 / w + 2 + 2; /* output rows a tile can touch, plus one above and below */
    const long floats = 3 * rows * (w + 8);
    if (floats > DN_PATCH_FLOATS) return 0;
    /* the copy moves whole wave-loads of 256 floats */
    return floats < DN_PATCH_MIN_FLOATS ? DN_PATCH_MIN_FLOATS : (floats + 255) / 256 * 256;
}

/* ---- weight packing ---------------------------------------------------------------------- */
/* taps > 0 selects the tap-blocked order (taps = size*size, c % 16 == 0): packed row k' holds
 * channel (k'/16/taps)*16 + k'%16 of tap (k'/16) % taps; taps == 0 keeps the reference order. */
__global__ void pack_weights_kernel(const float *w, float *packed, int M, int K, int Mpad, long total, int taps)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        /* packed index = ((chunk*4 + slot)*Mpad + m)*4 + j,  position in chunk kk = 4*slot + j */
        const int j = (int)(i & 3);
        long t = i >> 2;
        const int m = (int)(t % Mpad);
        t /= Mpad;
        const int q = (int)(t & 3);
        const int kc = (int)(t >> 2);
        const int kk = q * 4 + j;
        int k = kc * DN_BK + kk;
        if (taps > 0) {
            const int cb = kc / taps, tap = kc - cb * taps;
            k = (cb * DN_BK + kk) * taps + tap;
        }
        packed[i] = (m < M && k < K) ? w[(long)m * K + k] : 0.f;
    }
}

/* Grouped layers whose groups have as many filters as channels, at most 32 of each (ResNeXt's
 * 32-group 3x3: 4, 8, 16 or 32 per group): filters [32t, 32t+32) then read exactly input
 * channels [32t, 32t+32), so tile t is a dense 32 x (32*taps) GEMM over those channels with
 * block-diagonal weights (zeros between groups).  The zeros cost 32/cg times the layer's nominal
 * FLOPs on the matrix cores, which is still 10-50x less time than a per-group direct loop, and
 * nothing at all at 32 channels per group.  Returns taps (9 or 1), 0 if the layer does not fit. */
static inline int conv_grouped_tile(int n, int c, int groups, int size)
{
    if (groups <= 1 || n % groups || c % groups) return 0;
    const int cg = c / groups, fg = n / groups;
    if (cg != fg || cg > 32 || (32 % cg) != 0 || (n % 32) != 0) return 0;
    if (size == 3) return 9;
    if (size == 1) return 1;
    return 0;
}

/* packed[((tile*KCH + chunk)*4 + slot)*32 + r][j]: filter 32*tile + r, tap-blocked k inside the
 * tile's 32 channels; weights are [n][cg][size*size] */
__global__ void pack_grouped_kernel(const float *w, float *packed, int cg, int taps, long total)
{
    const int kch = 2 * taps;
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const int j = (int)(i & 3);
        long t = i >> 2;
        const int r = (int)(t & 31);
        t >>= 5;
        const int q = (int)(t & 3);
        t >>= 2;
        const int kc = (int)(t % kch);
        const int tile = (int)(t / kch);
        const int cb = kc / taps, tap = kc - cb * taps;
        const int ch = cb * DN_BK + q * 4 + j;  /* channel inside the tile, 0..31 */
        const int f = tile * 32 + r;             /* filter */
        const bool same_group = (r / cg) == (ch / cg);
        packed[i] = same_group ? w[((long)f * cg + (ch % cg)) * taps + tap] : 0.f;
    }
}

/* K order of a layer, from the layer geometry alone so that packing and forward agree. */
static inline int tap_blocked_taps(int c, int groups, int size)
{
    if (groups != 1 || (c % DN_BK) != 0) return 0;
    if (size == 1) return 1;
    if (size == 3) return 9;
    return 0;
}

/* fp32 part of the packed buffer */
static size_t conv_packed_f32_floats(int n, int c, int groups, int size)
{
    const int gt = conv_grouped_tile(n, c, groups, size);
    if (gt) return (size_t)(n / 32) * (size_t)(2 * gt) * DN_BK * 32;
    if (groups != 1) return 0;
    const long K = (long)c * size * size;
    const long kch = (K + DN_BK - 1) / DN_BK;
    const long mpad = ((long)n + DN_MPAD - 1) / DN_MPAD * DN_MPAD;
    return (size_t)(kch * mpad * DN_BK);
}

/* Rows of the bf16 copy: whole 256-row tiles for layers that use them, else as the fp32 part. */
static int conv_mpad16(int n)
{
    const int unit = n > 128 ? 256 : DN_MPAD;
    return (n + unit - 1) / unit * unit;
}

/* bf16 part (tap-blocked and grouped layers only), counted in floats: it follows the fp32 part in
 * the same buffer so that one pointer still stands for a layer's packed weights */
static size_t conv_packed_bf16_floats(int n, int c, int groups, int size)
{
    const int gt = conv_grouped_tile(n, c, groups, size);
    if (gt) return conv_packed_f32_floats(n, c, groups, size) / 2;
    const int taps = tap_blocked_taps(c, groups, size);
    if (!taps) return 0;
    const long kch = (long)c * taps / DN_BK;
    return (size_t)(kch * conv_mpad16(n) * DN_BK / 2);
}

/* three bf16 copies follow the fp32 part: hi (the bf16 mode's operand), then mid and lo, which the
 * three-piece emulation adds */
#define DN_BF16_PLANES 3

extern "C" size_t conv_packed_floats(int n, int c, int groups, int size)
{
    return conv_packed_f32_floats(n, c, groups, size) + DN_BF16_PLANES * conv_packed_bf16_floats(n, c, groups, size);
}

/* piece `plane` of w = hi + mid + lo, each the nearest-even bf16 of what the previous ones left */
__device__ __forceinline__ __bf16 conv_bf16_piece(float w, int plane)
{
    __bf16 p = (__bf16)w;
    for (int i = 0; i < plane; ++i) {
        w -= (float)p; /* exact */
        p = (__bf16)w;
    }
    return p;
}

/* bf16 copy of a tap-blocked layer: element ((chunk*2 + h)*Mpad16 + m)*8 + p is the weight that the
 * fp32 layout keeps at slot (p < 4 ? h : 2 + h), position p % 4 of the same chunk and row (1x1
 * layers) or at position 8*h + p of the chunk (3x3 layers), rounded to nearest even. */
__global__ void pack_weights_bf16_kernel(const float *w, __bf16 *packed, int M, int K, int Mpad16, long total, int taps,
                                         int plane)
{
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const int pp = (int)(i & 7);
        long t = i >> 3;
        const int m = (int)(t % Mpad16);
        t /= Mpad16;
        const int h = (int)(t & 1);
        const int kc = (int)(t >> 1);
        /* 1x1: the order the fp32 activation slots give (slot h, then slot 2 + h); 3x3: the staged
         * input's, eight consecutive channels per half */
        const int kk = taps == 1 ? (pp < 4 ? h : 2 + h) * 4 + (pp & 3) : 8 * h + pp;
        const int cb = kc / taps, tap = kc - cb * taps;
        const int k = (cb * DN_BK + kk) * taps + tap;
        packed[i] = conv_bf16_piece((m < M && k < K) ? w[(long)m * K + k] : 0.f, plane);
    }
}

/* bf16 copy of a grouped layer: ((tile*KCH + chunk)*2 + h)*32 + r rows of 8, as above */
__global__ void pack_grouped_bf16_kernel(const float *w, __bf16 *packed, int cg, int taps, long total, int plane)
{
    const int kch = 2 * taps;
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const int pp = (int)(i & 7);
        long t = i >> 3;
        const int r = (int)(t & 31);
        t >>= 5;
        const int h = (int)(t & 1);
        t >>= 1;
        const int kc = (int)(t % kch);
        const int tile = (int)(t / kch);
        const int cb = kc / taps, tap = kc - cb * taps;
        const int ch = cb * DN_BK + (taps == 1 ? (pp < 4 ? h : 2 + h) * 4 + (pp & 3) : 8 * h + pp);
        const int f = tile * 32 + r;
        const bool same_group = (r / cg) == (ch / cg);
        packed[i] = conv_bf16_piece(same_group ? w[((long)f * cg + (ch % cg)) * taps + tap] : 0.f, plane);
    }
}

static inline int pack_blocks(size_t total)
{
    const size_t b = (total + 255) / 256;
    return (int)(b > 8192 ? 8192 : b);
}

extern "C" void conv_pack_weights_gpu(const float *weights, float *packed, int n, int c, int groups, int size)
{
    const size_t total = conv_packed_f32_floats(n, c, groups, size);
    if (!total || hip_parse_only()) return;
    const size_t total16 = conv_packed_bf16_floats(n, c, groups, size) * 2; /* bf16 elements */
    __bf16 *packed16 = (__bf16 *)(packed + total);
    const int gt = conv_grouped_tile(n, c, groups, size);
    if (gt) {
        hipLaunchKernelGGL(pack_grouped_kernel, dim3(pack_blocks(total)), dim3(256), 0, dn_stream(), weights, packed,
                           c / groups, gt, (long)total);
        for (int pl = 0; pl < DN_BF16_PLANES; ++pl)
            hipLaunchKernelGGL(pack_grouped_bf16_kernel, dim3(pack_blocks(total16)), dim3(256), 0, dn_stream(), weights,
                               packed16 + (size_t)pl * total16, c / groups, gt, (long)total16, pl);
        dn_check_launch("conv_pack_weights_gpu");
        return;
    }
    const int K = c * size * size;
    const int mpad = (n + DN_MPAD - 1) / DN_MPAD * DN_MPAD;
    const int taps = tap_blocked_taps(c, groups, size);
    hipLaunchKernelGGL(pack_weights_kernel, dim3(pack_blocks(total)), dim3(256), 0, dn_stream(), weights, packed, n,
                       K, mpad, (long)total, taps);
    for (int pl = 0; total16 && pl < DN_BF16_PLANES; ++pl)
        hipLaunchKernelGGL(pack_weights_bf16_kernel, dim3(pack_blocks(total16)), dim3(256), 0, dn_stream(), weights,
                           packed16 + (size_t)pl * total16, n, K, conv_mpad16(n), (long)total16, taps, pl);
    dn_check_launch("conv_pack_weights_gpu");
}

/* ---- bf16 staging of a 3x3 layer's input -------------------------------------------------- */
/* [image][C][H*W] fp32 -> [image][C/8][H*W] rows of eight bf16 (nearest even): one thread per
 * output row; for each of its eight channels consecutive threads read consecutive pixels, and
 * they write consecutive 16-byte rows. */
__global__ void stage_bf16_kernel(const float *in, bf16x8 *out, int cblocks, int HW, long total)
{
    const long i = blockIdx.x * (long)blockDim.x + threadIdx.x;
    if (i >= total) return;
    const long img_blk = i / HW;                 /* image * cblocks + block */
    const int pix = (int)(i - img_blk * HW);
    const float *src = in + img_blk * 8 * HW + pix;
    f32x8 f;
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = src[(long)j * HW];
    out[i] = __builtin_convertvector(f, bf16x8);
}

static float *g_stage = 0; /* staged input of the bf16 3x3 path, grown on demand */
static size_t g_stage_floats = 0;

/* ---- dispatch ---------------------------------------------------------------------------- */
/* One-shot kernel timing: the next MFMA convolution launches its main kernel with these two
 * events attached to the dispatch itself (start and end of the kernel as the GPU stamps them,
 * no extra packets on the stream), then forgets them. */
static hipEvent_t g_prof_start = 0, g_prof_stop = 0;
extern "C" void conv_profile_next(void *start_event, void *stop_event)
{
    g_prof_start = (hipEvent_t)start_event;
    g_prof_stop = (hipEvent_t)stop_event;
}
extern "C" int conv_profile_pending(void) { return g_prof_start != 0; }

static int g_algo = 0;
static int g_cus = 0; /* compute units of the current device (conv_device_setup) */
/* Tuning and test hooks of the K-split (conv_set_ksplit): 0 / default = automatic. */
static int g_tune_split = 0;   /* > 0: this many slices for every tail tile (1 = none) */
static int g_tune_bn = 0;      /* 64 or 128: column width of the 128-row fp32 tile */
extern "C" void conv_set_algo(int algo) { g_algo = algo; }

/* 0 = fp32 operands (default, the reference's arithmetic); 1 = the tap-blocked MFMA kernels round
 * both operands to bf16 and accumulate in fp32; 2 = they split both operands into three bf16 pieces
 * and sum six piece-products in fp32 (fp32-level accuracy on the bf16 matrix cores).  Layers on
 * other kernels stay fp32. */
static int g_precision = 0;

/* Whether a layer of conv_mode `mode` goes to the first-layer kernel when its geometry fits: the
 * 3-channel layers of the reference-order mode, and 16-channel 3x3 layers of the tap-blocked mode
 * while the operands are fp32 (the bf16 modes keep such a layer on their own pipeline). */
static int conv_first_takes(int mode, int c)
{
    if (g_algo != 0) return 0;
    return (mode == 3 && c == 3) || (mode == 13 && c == 16 && g_precision == 0);
}

/* Whether a grouped layer goes to the vector-ALU kernel of small groups when its geometry fits: in
 * the default mode only (conv_set_algo(3) keeps such a layer on the matrix cores: the cross-check). */
static int conv_group_takes(void) { return g_algo == 0 && g_precision == 0; }

extern "C" void conv_set_precision(int precision)
{
    if (precision < 0 || precision > 2)
        dn_fatal("conv_set_precision: 0 (fp32), 1 (bf16 operands) or 2 (fp32 emulated with three bf16 pieces)");
    g_precision = precision;
}
extern "C" int conv_get_precision(void) { return g_precision; }

static int conv_mode(int c, int groups, int size, int stride, int pad, long in_bytes);

/* Layers with more than 64 filters run 128x128 tiles, or 128x64 tiles when the layer has fewer
 * 128-wide tiles than the chip has CUs (batch 1): twice the workgroups before any cut along K,
 * and fewer padded columns (192 instead of 256 for the 169 pixels of a 13x13 image).  Measured on
 * every such layer of yolov3 at batch 1: 8-25% less time than the wide tile at its best split. */
/* 64x64 tiles (four waves of 32x32, eight workgroups per CU) for layers of 33..64 filters and for
 * 1x1 layers of any more: with so little K per tile (16..64 chunks) the load latency at the start
 * of a tile and its epilogue weigh as much as the MFMAs, and many small workgroups per CU overlap
 * them better than three large ones.  Measured at batch 64 (min of three interleaved runs): 3x3
 * 32->64 at 208x208 898 against 974 microseconds with 64x256 tiles, 1x1 128->64 at 104x104 137
 * against 161, 1x1 1024->512 at 13x13 104 against 112; at batch 1 (tiles fewer than CUs) 23 instead
 * of 34-37 microseconds for the 3x3 32->64 layers and 9-10 instead of 11-12 for the 1x1 layers. */
static bool conv_small_tile(long columns, int n, int kch, int size)
{
    (void)columns;
    (void)kch;
    if (g_tune_bn) return g_tune_bn == 1 || (g_tune_bn == 64 && n <= 64);
    return n <= 64 || size == 1;
}

/* 128x64 tiles (five workgroups per CU against four of 128x128) for 3x3 layers of 128 to 256 input
 * channels, and for any layer whose 128x128 tiles would number fewer than the CUs.  Measured at batch
 * 64, narrow against wide, microseconds: 706 / 718 for 256->512 at 26x26, 713 / 719 for 128->256 at
 * 52x52, 747 / 759 for 128->256 stride 2 at 104x104; but 753 / 737 for 64->128 at 104x104 (twice the
 * prologues and epilogues per MFMA weigh more on a short K) and 740 / 728 for 512->1024 at 13x13
 * (every tile streams 18 MB of weights, the narrow one twice as often per output). */
static bool conv_narrow_tile(long columns, int n, int kch, int size)
{
    if (g_tune_bn) return g_tune_bn == 64;
    if (size == 3 && kch >= 72 && kch <= 144) return true;
    const long tiles = ((columns + 127) / 128) * ((n + 127) / 128);
    return tiles < 256;
}

static const char *kernel_name(int n, int c, int groups, int size, long columns, int patch, int mode);

/* Without the layer's geometry the first-layer kernel cannot be told from the generic one: the name
 * assumes stride 1, pad size/2 and never names conv_patch_kernel (conv_kernel_name_geometry does). */
extern "C" const char *conv_kernel_name_columns(int n, int c, int groups, int size, long columns)
{
    int mode = conv_mode(c, groups, size, 1, size / 2, 0);
    if (conv_grouped_tile(n, c, groups, size) && g_algo != 1) mode = 10 + size;
    return kernel_name(n, c, groups, size, columns, 0, mode);
}

/* The name for a whole layer, decided by the predicates the dispatch itself uses (conv_forward). */
extern "C" const char *conv_kernel_name_geometry(int batch, int c, int h, int w, int n, int groups, int size,
                                                 int stride, int pad)
{
    const int out_h = (h + 2 * pad - size) / stride + 1, out_w = (w + 2 * pad - size) / stride + 1;
    /* a batch beyond the 32-bit offsets runs in slices of whole images */
    const long in_img = (long)c * h * w * 4;
    const long by_bytes = ((1L << 32) - (2L << 20)) / in_img, by_cols = ((1L << 31) - 1024) / ((long)out_h * out_w);
    const long per = by_bytes < by_cols ? by_bytes : by_cols;
    if (g_algo != 1 && per >= 1 && per < batch) batch = (int)per;
    const long columns = (long)batch * out_h * out_w;
    int mode = conv_mode(c, groups, size, stride, pad, (long)batch * in_img);
    if (g_algo != 1 && !(size == 3 && pad != 1) && conv_grouped_tile(n, c, groups, size)) mode = 10 + size;
    if (columns >= (1L << 31) - 512) mode = -1;
    if (conv_first_takes(mode, c) && conv_first_serves(batch, c, h, w, n, groups, size, stride, pad))
        return conv_first_kernel_name(c, n, 0, h, w);
    if (conv_group_takes() && conv_group_serves(batch, c, h, w, n, groups, size, stride, pad))
        return conv_group_kernel_name(c, groups, stride);
    const int patch = g_algo == 0 && mode == 3 && conv_patch_floats(c, h, w, n, groups, size, stride, pad) > 0;
    return kernel_name(n, c, groups, size, columns, patch, mode);
}

static const char *kernel_name(int n, int c, int groups, int size, long columns, int patch, int mode)
{
    static char name[96];
    int bm = n <= 32 ? 32 : n <= 64 ? 64 : 128;
    if (mode >= 10 && groups > 1) bm = 32;
    if (mode < 0) return "conv_direct_kernel";
    if (patch) return n <= 32 ? "conv_patch_kernel<1,3>" : "conv_patch_kernel<2,3>";
    const int bf16 = g_precision == 1 && mode >= 10;
    const int x3 = g_precision == 2 && mode >= 10;
    if (bf16 && bm == 128 && n > 128) bm = 256;
    if (x3 && bm == 128)
        snprintf(name, sizeof name, "conv_mfma_kernel<128,128,128,32,%d,3>", mode);
    else if (bm == 128 && g_precision == 0 && columns > 0 && conv_small_tile(columns, n, (c * size * size + 15) / 16, size))
        snprintf(name, sizeof name, "conv_mfma_kernel<64,64,32,32,%d>", mode);
    else if (bm == 128 && g_precision == 0 && columns > 0 && conv_narrow_tile(columns, n, (c * size * size + 15) / 16, size)) {
        const long tiles = ((columns + 63) / 64) * ((n + 127) / 128);
        const int sparse = tiles < (g_cus > 0 ? g_cus : 256) && mode >= 11; /* the variant of launches that do not fill the chip */
        snprintf(name, sizeof name, "conv_mfma_kernel<128,64,64,32,%d>", mode + 100 * sparse);
    }
    else if (bm == 64 && g_precision == 0 && columns > 0 && conv_small_tile(columns, n, (c * size * size + 15) / 16, size))
        snprintf(name, sizeof name, "conv_mfma_kernel<64,64,32,32,%d>", mode);
    else
        snprintf(name, sizeof name, "conv_mfma_kernel<%d,%d,%d,64,%d%s>", bm, bm >= 128 ? 128 : 256,
                 bm == 32 ? 32 : bm == 256 ? 128 : 64, mode, x3 ? ",3" : !bf16 ? "" : mode == 13 ? ",2" : ",1");
    return name;
}

extern "C" const char *conv_kernel_name(int n, int c, int groups, int size)
{
    return conv_kernel_name_columns(n, c, groups, size, -1); /* size of the layer unknown: the large-layer kernel */
}

static float *g_scratch = 0;       /* per-call repack buffer for callers without a packed copy */
static size_t g_scratch_floats = 0;

static float *g_partial = 0; /* K-slice accumulators of tail tiles, grown on demand */
static size_t g_partial_floats = 0;

/* ---- allocation-free calls ----------------------------------------------------------------
 * forward_convolutional_noalloc_gpu serves callers that cannot allocate device memory (stream
 * capture, tight serving loops).  The only device memory a packed-weights fp32 call needs beyond
 * its operands is the K-slice accumulator buffer above; for these calls it is a fixed array in
 * the code object.  `scratch` is the host-side handle of that array, not an address: host code
 * uses the per-device pointer hipGetSymbolAddress returns (every device holds its own copy). */
#define DN_NOALLOC_SCRATCH_FLOATS ((size_t)16 << 20) /* 64 MiB */
#define DN_MAX_DEVICES 16
static __device__ __align__(256) float scratch[DN_NOALLOC_SCRATCH_FLOATS];
static float *g_scratch_dev[DN_MAX_DEVICES];
static int g_cus_dev[DN_MAX_DEVICES];
static int g_noalloc = 0;       /* inside forward_convolutional_noalloc_gpu */
static int g_noalloc_error = 0; /* set instead of allocating (or launching) by the paths below */

/* Once per device, with that device current: address of its copy of `scratch`, CU count. */
extern "C" __attribute__((visibility("hidden"))) void conv_device_setup(void)
{
    if (hip_parse_only()) return;
    const int dev = hip_get_device();
    if (dev < 0 || dev >= DN_MAX_DEVICES) dn_fatal("conv_device_setup: device index out of range");
    if (!g_scratch_dev[dev]) {
        float *ptr = 0;
        hip_check_error(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) dn_fatal("conv_device_setup: hipGetSymbolAddress returned a null pointer");
        g_scratch_dev[dev] = ptr;
    }
    if (!g_cus_dev[dev]) {
        hipDeviceProp_t prop;
        hip_check_error(hipGetDeviceProperties(&prop, dev));
        g_cus_dev[dev] = prop.multiProcessorCount;
    }
    conv_first_device_setup(); /* resident workgroups per CU of the first-layer kernels */
}

static int g_tune_bands = 0;
extern "C" void conv_set_bands(int bands) { g_tune_bands = bands; }

extern "C" void conv_set_ksplit(int split, int tile_n)
{
    if (split < -32 || (tile_n != 0 && tile_n != 1 && tile_n != 64 && tile_n != 128))
        dn_fatal("conv_set_ksplit: split >= 0, tile_n 0, 1, 64 or 128");
    g_tune_split = split;
    g_tune_bn = tile_n;
}

/* The K-slice accumulator buffer for `need` floats: the growing allocation, or in an
 * allocation-free call the current device's fixed array (null when it is too small). */
static float *partial_buffer(size_t need)
{
    if (g_noalloc) {
        if (need > DN_NOALLOC_SCRATCH_FLOATS) {
            fprintf(stderr,
                    "forward_convolutional_noalloc_gpu: this geometry needs %zu bytes of K-split scratch, the fixed "
                    "buffer holds %zu\n", need * sizeof(float), DN_NOALLOC_SCRATCH_FLOATS * sizeof(float));
            g_noalloc_error = 1;
            return 0;
        }
        return g_scratch_dev[hip_get_device()];
    }
    if (need > g_partial_floats) {
        if (g_partial) hip_free(g_partial);
        g_partial = hip_make_array(0, need);
        g_partial_floats = need;
    }
    return g_partial;
}

/* How to cover `tiles` equal tiles on `cus` compute units.  Whole tiles are dealt out in rounds;
 * a remainder that would leave most CUs idle for a whole tile time (or, at batch 1, a grid far
 * smaller than the chip) is cut along K into `split` slices each, which conv_reduce_kernel sums.
 * Returns the number of whole tiles; *split = 1 means no tail. */
static long plan_split(long tiles, int kch, int cus, int *split, double fixed_scale, int bm, int bn)
{
    *split = 1;
    if (g_algo == 3 || cus <= 0) return tiles;
    if (g_tune_split < 0) { /* tuning hook: every tile cut into -split slices */
        *split = -g_tune_split < kch ? -g_tune_split : kch;
        return *split > 1 ? 0 : tiles;
    }
    const long whole = tiles / cus * cus;
    const long tail = tiles - whole;
    if (tail == 0) return tiles;
    if (g_tune_split > 0) {
        *split = g_tune_split < kch ? g_tune_split : kch;
        return *split > 1 ? whole : tiles;
    }
    if (tail * 10 >= (long)cus * 9) return tiles; /* a nearly full round: leave it */
    if (whole == 0 && (fixed_scale == 1.0 || bn == 64)) {
        /* The layer does not fill the chip even once (batch 1).  Times in microseconds, fitted to a
         * sweep of the split factor over the layers of yolov3 at batch 1: a workgroup alone on its
         * CU cannot hide its LDS reads and barriers behind another one's MFMAs and takes `lone`
         * per 16-wide chunk, r workgroups sharing a CU take r * `shared`; an unsplit tile pays its
         * epilogue (2.4), a split one the second launch (5) and, per slice, the extra partial
         * traffic of both launches. */
        const double work = (double)bm * bn / (128.0 * 128.0); /* MFMAs per chunk against the 128x128 tile */
        const double lone = work <= 0.25 ? 0.28 : work <= 0.5 ? 0.55 : 1.1, shared = work <= 0.25 ? 0.23 : work <= 0.5 ? 0.45 : 0.9,
                     per_slice = work <= 0.25 ? 0.22 : work <= 0.5 ? 0.4 : 0.8;
        double best = kch * lone + 2.4;
        const int max_s = kch / 2 < 32 ? kch / 2 : 32;
        for (int s = 2; s <= max_s; ++s) {
            const long r = (tail * s + cus - 1) / cus; /* workgroups per CU */
            const double chunks = (double)kch / s;
            const double cost = chunks * (r == 1 ? lone : shared * (double)r) + 5.0 + per_slice * s;
            if (cost < 0.92 * best) {
                best = cost / 0.92; /* later candidates must beat this one outright */
                *split = s;
            }
        }
        return *split > 1 ? whole : tiles;
    }
    /* Time in units of one 16-wide K chunk.  A workgroup costs its chunks plus a fixed part
     * (first load latency, epilogue or partial store); the reduce pass costs a little more. */
    const double fixed_whole = 5.0 * fixed_scale, fixed_slice = 8.0 * fixed_scale, reduce = 4.0 * fixed_scale;
    double best = (double)kch + fixed_whole;                   /* the tail as whole tiles */
    const int max_s = kch / 4 < 32 ? kch / 4 : 32;             /* at least 4 chunks per slice */
    for (int s = 2; s <= max_s; ++s) {
        const long rounds = (tail * s + cus - 1) / cus;
        const double cost = rounds * ((double)kch / s + fixed_slice) + reduce;
        if (cost < 0.9 * best) {
            best = cost / 0.9;                                 /* later candidates must beat this one outright */
            *split = s;
        }
    }
    return *split > 1 ? whole : tiles;
}

typedef void (*conv_kernel_t)(mfma_args);

/* The kernel instance for a tile shape, K order and precision; null when it is not built. */
template <int BM, int BN, int WM, int WN>
static conv_kernel_t pick_kernel(int mode, int bf16, int x3, int sparse)
{
    constexpr bool X3_ONLY = WM == 128 && WN == 32; /* the 128x32 wave tile is built for the three-piece mode alone ... */
    constexpr bool NO_X3 = BM == 128 && WN == 64;   /* ... which never runs the 128x128 tile with 64x64 wave tiles */
    constexpr bool FP32_ONLY = BN == 64;            /* the narrow tile of small layers */
    if (BM > 128 && !bf16) dn_fatal("conv dispatch: the 256-row tile is only built for the bf16-operand mode");
    if (NO_X3 && x3) dn_fatal("conv dispatch: the three-piece mode runs 128x128 tiles with 128x32 wave tiles");
    if (X3_ONLY && !x3) dn_fatal("conv dispatch: the 128x32 wave tile is only built for the three-piece mode");
    if (FP32_ONLY && (bf16 || x3)) dn_fatal("conv dispatch: the 64-column tiles are only built for fp32 operands");
    if constexpr (FP32_ONLY) {
        if constexpr (BM == 128) {
            if (sparse && mode == 11) return conv_mfma_kernel<BM, BN, WM, WN, 111>;
            if (sparse && mode == 13) return conv_mfma_kernel<BM, BN, WM, WN, 113>;
        }
        switch (mode) {
        case 11: return conv_mfma_kernel<BM, BN, WM, WN, 11>;
        case 13: return conv_mfma_kernel<BM, BN, WM, WN, 13>;
        case 1: return conv_mfma_kernel<BM, BN, WM, WN, 1>;
        case 3: return conv_mfma_kernel<BM, BN, WM, WN, 3>;
        case 7: return conv_mfma_kernel<BM, BN, WM, WN, 7>;
        default: return conv_mfma_kernel<BM, BN, WM, WN, 0>;
        }
    } else {
        switch (mode) {
        case 11:
            if constexpr (X3_ONLY) return conv_mfma_kernel<BM, BN, WM, WN, 11, 3>;
            else if (bf16) return conv_mfma_kernel<BM, BN, WM, WN, 11, 1>;
            else if constexpr (BM <= 128) {
                if constexpr (!NO_X3)
                    if (x3) return conv_mfma_kernel<BM, BN, WM, WN, 11, 3>;
                return conv_mfma_kernel<BM, BN, WM, WN, 11>;
            }
            break;
        case 13:
            if constexpr (X3_ONLY) return conv_mfma_kernel<BM, BN, WM, WN, 13, 3>;
            else if (bf16) return conv_mfma_kernel<BM, BN, WM, WN, 13, 2>;
            else if constexpr (BM <= 128) {
                if constexpr (!NO_X3)
                    if (x3) return conv_mfma_kernel<BM, BN, WM, WN, 13, 3>;
                return conv_mfma_kernel<BM, BN, WM, WN, 13>;
            }
            break;
        default:
            if constexpr (BM <= 128 && !X3_ONLY) {
                if (mode == 1) return conv_mfma_kernel<BM, BN, WM, WN, 1>;
                if (mode == 3) return conv_mfma_kernel<BM, BN, WM, WN, 3>;
                if (mode == 7) return conv_mfma_kernel<BM, BN, WM, WN, 7>;
                return conv_mfma_kernel<BM, BN, WM, WN, 0>;
            }
            break;
        }
    }
    return 0;
}

template <int BM, int BN, int WM, int WN>
static void launch_tile(const mfma_args &a0, int mode)
{
    mfma_args a = a0;
    a.tiles_m = (a.M + BM - 1) / BM;
    a.tiles_n = (int)((a.Ntotal + BN - 1) / BN);
    const long total = (long)a.tiles_m * a.tiles_n;
    /* Bands of filter tiles.  Every XCD has a private L2, so with one band (filter tile fastest over
     * the whole layer) each of the eight reads all the weights and one eighth of the input; with b
     * bands an XCD reads 1/b of the weights and the input b/8 times.  The count that minimises
     * weights*8/b + input*b wins (measured with the L2 fetch counter on 3x3 512->1024 at 13x13,
     * batch 64: 173 MB with one band, 120 MB with four, and 2% less time). */
    int bands = 1;
    if (g_tune_bands > 0)
        bands = g_tune_bands;
    else if (total < 256)
        bands = 8; /* a launch that does not fill the chip is bound by latency: the fewer distinct weight
                    * bytes an XCD pulls in, the better (3x3 256->512 at 26x26, batch 1: 26.9 against 30.0 us) */
    else {
        double best = 8.0 * a.wp_records + a.in_records;
        for (int b = 2; b <= 8; b <<= 1) {
            const double cost = 8.0 * a.wp_records / b + (double)a.in_records * b;
            if (a.tiles_m % b == 0 && cost < 0.9 * best) best = cost, bands = b;
        }
    }
    while (bands > 1 && a.tiles_m % bands) bands >>= 1;
    a.m_group = a.tiles_m / bands;
    a.band_tiles = a.m_group * a.tiles_n;
    const int dev = hip_get_device();
    if (dev < 0 || dev >= DN_MAX_DEVICES) dn_fatal("conv dispatch: device index out of range");
    if (!g_cus_dev[dev]) conv_device_setup();
    g_cus = g_cus_dev[dev];
    const int bf16 = g_precision == 1 && mode >= 10;
    const int x3 = g_precision == 2 && mode >= 10;
    int split = 1;
    /* a bf16 chunk takes a small fraction of an fp32 chunk's time; the fixed costs do not shrink */
    /* ... and a chunk of a 64-column tile is half or a quarter of the 128x128 chunk the fixed costs are counted in */
    const long whole = plan_split(total, a.KCH, g_cus, &split, bf16 ? 6.0 : x3 ? 2.0 : BN == 64 ? 16384.0 / (BM * BN) : 1.0, BM, BN);
    const long tail = total - whole;
    const conv_kernel_t kernel = pick_kernel<BM, BN, WM, WN>(mode, bf16, x3, total < g_cus);
    if (!kernel) dn_fatal("conv dispatch: no kernel for this tile shape and mode");
    a.whole_tiles = (int)whole;
    a.split = split;
    a.per_xcd = (int)((whole + 7) / 8);
    a.partial = 0;
    if (tail > 0) {
        a.partial = partial_buffer((size_t)tail * split * BM * BN);
        if (!a.partial) return; /* allocation-free call and the fixed buffer is too small: nothing is launched */
    }
    const dim3 grid((unsigned)(a.per_xcd * 8 + tail * split));
    void *args[] = {&a};
    if (g_prof_start)
        hip_check_error(hipExtLaunchKernel((const void *)kernel, grid, dim3(DN_THREADS), args, 0, dn_stream(), g_prof_start,
                                           g_prof_stop, 0));
    else
        hip_check_error(hipLaunchKernel((const void *)kernel, grid, dim3(DN_THREADS), args, 0, dn_stream()));
    g_prof_start = g_prof_stop = 0;
    if (tail > 0)
        hipLaunchKernelGGL((conv_reduce_kernel<BM, BN, WM, WN>), dim3((unsigned)(tail * (BM * BN / 4 / DN_THREADS))),
                           dim3(DN_THREADS), 0, dn_stream(), a);
}

/* Which kernel variant serves a geometry: -1 = direct kernel, else the MODE template value. */
static int conv_mode(int c, int groups, int size, int stride, int pad, long in_bytes)
{
    const long K = (long)(c / (groups > 0 ? groups : 1)) * size * size;
    if (groups != 1 || g_algo == 1 || (size == 3 && K >= 32768)) return -1;
    /* the gather addresses the input through 32-bit buffer offsets */
    if (in_bytes + (1L << 20) >= (1L << 32)) return -1;
    const int taps = tap_blocked_taps(c, groups, size);
    if (taps) {
        /* the tap-blocked kernel needs pad 1 for 3x3; weights of such layers are packed
         * tap-blocked, so the rare misfit goes to the direct kernel rather than to the generic
         * MFMA kernel, which expects the reference K order */
        if (size == 3 && pad != 1) return -1;
        return 10 + size;
    }
    return size == 1 ? 1 : size == 3 ? 3 : size == 7 ? 7 : 0;
}

extern "C" void forward_shortcut_gpu(const float *, const float *, float *, int, int, int, int, int, int, int,
                                     float, float, int);
extern "C" void forward_yolo_gpu(const float *, float *, int, int, int, int, int);
extern "C" void dn_activate_array(float *x, long n, int activation);

static void conv_forward(const float *input, const float *weights, const float *packed, const float *biases,
                         const float *scales, const float *rolling_mean, const float *rolling_variance,
                         float *output, int batch, int c, int h, int w, int n, int groups, int size, int stride,
                         int pad, int batch_normalize, int activation, const float *add, float *sum, float s1,
                         float s2, int sum_act, int yolo_entries)
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

    /* The MFMA kernels address the input through 32-bit buffer offsets and count output columns in
     * 32 bits.  A batch beyond that is processed in slices of whole images (images are independent),
     * so only a single image of 4 GiB or 2^31 pixels ever falls back to the direct kernel. */
    if (g_algo != 1 && batch > 1) {
        const long in_img = (long)c * h * w * 4, out_img = (long)n * oh * ow;
        const long by_bytes = ((1L << 32) - (2L << 20)) / in_img, by_cols = ((1L << 31) - 1024) / ((long)oh * ow);
        const long per = by_bytes < by_cols ? by_bytes : by_cols;
        if (per >= 1 && per < batch) {
            for (long b0 = 0; b0 < batch; b0 += per) {
                const int nb = (int)(batch - b0 < per ? batch - b0 : per);
                conv_forward(input + b0 * (in_img / 4), weights, packed, biases, scales, rolling_mean, rolling_variance,
                             output + b0 * out_img, nb, c, h, w, n, groups, size, stride, pad, batch_normalize,
                             activation, add ? add + b0 * out_img : 0, sum ? sum + b0 * out_img : 0, s1, s2, sum_act,
                             yolo_entries);
                if (g_noalloc_error) return;
            }
            return;
        }
    }

    const long K = (long)(c / groups) * size * size;
    int mode = conv_mode(c, groups, size, stride, pad, (long)batch * c * h * w * 4);
    /* grouped layers that fit the 32-filter block-diagonal scheme run on the tap-blocked kernel */
    const int gtaps = (g_algo != 1 && (long)batch * c * h * w * 4 + (1L << 20) < (1L << 32) &&
                       !(size == 3 && pad != 1)) ? conv_grouped_tile(n, c, groups, size) : 0;
    if (gtaps) mode = 10 + size;
    if ((long)batch * oh * ow >= (1L << 31) - 512) mode = -1; /* the MFMA kernels index columns in 32 bits */
    if (mode < 0) {
        conv_direct_forward(input, weights, biases, scales, rolling_mean, rolling_variance, output, batch, c,
                            h, w, n, groups, size, stride, pad, batch_normalize, activation);
        if (sum && yolo_entries)
            forward_yolo_gpu(output, sum, batch, ow, oh, n / yolo_entries, yolo_entries - 5);
        else if (sum)
            forward_shortcut_gpu(output, add, sum, batch, ow, oh, n, ow, oh, n, s1, s2, sum_act);
        return;
    }
    double slope = 1., sum_slope = 1.;
    if (!conv_inline_activation(activation, &slope) ||
        (sum && !yolo_entries && !conv_inline_activation(sum_act, &sum_slope))) {
        /* an activation the epilogue does not carry: linear convolution, then the reference's own
         * sequence of passes (activate_array, src/convolutional_layer.c:478; shortcut) */
        conv_forward(input, weights, packed, biases, scales, rolling_mean, rolling_variance, output, batch, c, h,
                     w, n, groups, size, stride, pad, batch_normalize, DN_LINEAR, 0, 0, 0.f, 0.f, DN_LINEAR, 0);
        if (g_noalloc_error) return;
        dn_activate_array(output, (long)batch * n * oh * ow, activation);
        if (sum && yolo_entries)
            forward_yolo_gpu(output, sum, batch, ow, oh, n / yolo_entries, yolo_entries - 5);
        else if (sum)
            forward_shortcut_gpu(output, add, sum, batch, ow, oh, n, ow, oh, n, s1, s2, sum_act);
        return;
    }

    /* grouped 3x3 layers of 4 or 8 channels per group: the vector-ALU kernel (a block-diagonal tile on the
     * matrix cores would multiply 7/8 or 3/4 zeros) */
    if (conv_group_takes() && !sum && conv_group_serves(batch, c, h, w, n, groups, size, stride, pad)) {
        conv_group_forward(input, weights, biases, scales, rolling_mean, rolling_variance, output, batch, c, h, w, n,
                           groups, stride, batch_normalize, slope);
        return; /* a pending timing pair stays pending: conv_profile_pending() tells the caller it was not used */
    }
    /* first layers (3 channels, or 16 behind a pooled first layer; 3x3 / 1 / pad 1, even height, width a
     * multiple of 32): their own kernel */
    if (conv_first_takes(mode, c) && !sum && conv_first_serves(batch, c, h, w, n, groups, size, stride, pad)) {
        const int dev = hip_get_device();
        if (dev >= 0 && dev < DN_MAX_DEVICES && !g_cus_dev[dev]) conv_device_setup();
        conv_first_forward(input, weights, biases, scales, rolling_mean, rolling_variance, output, 0, 0, batch, c, h, w, n,
                           batch_normalize, slope, dev >= 0 && dev < DN_MAX_DEVICES ? g_cus_dev[dev] : 0,
                           (void *)g_prof_start, (void *)g_prof_stop);
        g_prof_start = g_prof_stop = 0;
        return;
    }
    const long patch = (g_algo == 0 && mode == 3 && !sum) ? conv_patch_floats(c, h, w, n, groups, size, stride, pad) : 0;
    if (g_noalloc && !patch && (!packed || (g_precision == 1 && mode == 13))) {
        fprintf(stderr, !packed ? "forward_convolutional_noalloc_gpu: this geometry runs on packed weights; pass the "
                                  "buffer conv_pack_weights_gpu wrote\n"
                                : "forward_convolutional_noalloc_gpu: the bf16-operand mode stages 3x3 inputs in a "
                                  "buffer it allocates; use conv_set_precision(0) or (2)\n");
        g_noalloc_error = 1;
        return;
    }
    if (!packed && !patch) {
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
    a.grouped = 0;
    if (gtaps && mode >= 10) { /* per 32-filter tile: 32 channels x taps */
        a.grouped = 1;
        a.K = 32 * gtaps;
        a.KCH = 2 * gtaps;
        a.Mpad = 32;
    }
    a.P = oh * ow;
    a.OW = ow;
    a.Ntotal = (long)batch * a.P;
    a.stride = stride;
    a.pad = pad;
    a.size = size;
    a.bn = batch_normalize ? 1 : 0;
    a.slope_hi = conv_split(slope).hi;
    a.slope_lo = conv_split(slope).lo;
    a.tiles_m = a.tiles_n = a.per_xcd = 0;
    a.m_group = a.band_tiles = 1;
    a.whole_tiles = 0;
    a.split = 1;
    a.partial = 0;
    a.add = add;
    a.sum = sum;
    a.yolo_entries = sum ? yolo_entries : 0;
    a.s1 = s1;
    a.s2 = s2;
    a.sum_slope_hi = conv_split(sum_slope).hi;
    a.sum_slope_lo = conv_split(sum_slope).lo;
    a.in_records = (unsigned)((long)batch * c * h * w * 4 + (long)(w + 1) * 4);
    a.wp_records = (unsigned)(conv_packed_f32_floats(n, c, groups, size) * 4);
    a.wp16 = packed + conv_packed_f32_floats(n, c, groups, size);
    a.plane16 = (unsigned)(conv_packed_bf16_floats(n, c, groups, size) * 4);
    a.wp16_records = DN_BF16_PLANES * a.plane16;
    a.Mpad16 = a.grouped ? 32 : conv_mpad16(n);
    a.in16 = 0;
    a.in16_records = 0;
    if (g_precision == 1 && mode == 13) {
        /* the 3x3 bf16 kernel gathers from a bf16 copy of the input, eight channels per 16 bytes */
        const long rows = (long)batch * (c / 8) * h * w;
        const size_t need = (size_t)rows * 4 + 64;
        if (need > g_stage_floats) {
            if (g_stage) hip_free(g_stage);
            g_stage = hip_make_array(0, need);
            g_stage_floats = need;
        }
        hipLaunchKernelGGL(stage_bf16_kernel, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, dn_stream(), input,
                           (bf16x8 *)g_stage, c / 8, h * w, rows);
        a.in16 = g_stage;
        a.in16_records = (unsigned)(rows * 16 + (long)(w + 1) * 16);
    }
    if (patch) {
        /* first layers (3 channels, 3x3): input rows through LDS, weights in registers */
        a.wp = weights;
        void *args[] = {&a};
        const void *kernel = n <= 32 ? (const void *)conv_patch_kernel<1, 3> : (const void *)conv_patch_kernel<2, 3>;
        const dim3 grid((unsigned)((long)batch * a.P / 256));
        if (g_prof_start)
            hip_check_error(hipExtLaunchKernel(kernel, grid, dim3(DN_THREADS), args, (size_t)patch * 4, dn_stream(),
                                               g_prof_start, g_prof_stop, 0));
        else
            hip_check_error(hipLaunchKernel(kernel, grid, dim3(DN_THREADS), args, (size_t)patch * 4, dn_stream()));
        g_prof_start = g_prof_stop = 0;
    } else if (n <= 32 || a.grouped)
        launch_tile<32, 256, 32, 64>(a, mode);
    else if (n > 128 && g_precision == 1 && mode >= 10)
        launch_tile<256, 128, 128, 64>(a, mode);
    else if (g_precision == 0 && conv_small_tile(a.Ntotal, n, a.KCH, size))
        launch_tile<64, 64, 32, 32>(a, mode);
    else if (n <= 64)
        launch_tile<64, 256, 64, 64>(a, mode);
    else if (g_precision == 2 && mode >= 10)
        /* four waves side by side, 128 rows x 32 columns each: no two waves split the same activations */
        launch_tile<128, 128, 128, 32>(a, mode);
    else if (g_precision == 0 && conv_narrow_tile(a.Ntotal, n, a.KCH, size))
        launch_tile<128, 64, 64, 32>(a, mode);
    else
        launch_tile<128, 128, 64, 64>(a, mode);
    dn_check_launch("forward_convolutional_gpu");
}

extern "C" void forward_convolutional_gpu(const float *input, const float *weights, const float *packed,
                                          const float *biases, const float *scales,
                                          const float *rolling_mean, const float *rolling_variance,
                                          float *output, int batch, int c, int h, int w, int n,
                                          int groups, int size, int stride, int pad,
                                          int batch_normalize, int activation)
{
    conv_forward(input, weights, packed, biases, scales, rolling_mean, rolling_variance, output, batch, c, h, w,
                 n, groups, size, stride, pad, batch_normalize, activation, 0, 0, 0.f, 0.f, DN_LINEAR, 0);
}

extern "C" void forward_convolutional_shortcut_gpu(const float *input, const float *weights, const float *packed,
                                                   const float *biases, const float *scales,
                                                   const float *rolling_mean, const float *rolling_variance,
                                                   float *output, int batch, int c, int h, int w, int n,
                                                   int groups, int size, int stride, int pad,
                                                   int batch_normalize, int activation, const float *add,
                                                   float *sum_output, float alpha, float beta,
                                                   int shortcut_activation)
{
    if (!add || !sum_output) dn_fatal("forward_convolutional_shortcut_gpu: null pointer");
    if (sum_output == output) dn_fatal("forward_convolutional_shortcut_gpu: sum_output must not alias output");
    if (shortcut_activation < 0 || shortcut_activation > DN_SELU)
        dn_fatal("forward_convolutional_shortcut_gpu: unknown activation");
    conv_forward(input, weights, packed, biases, scales, rolling_mean, rolling_variance, output, batch, c, h, w,
                 n, groups, size, stride, pad, batch_normalize, activation, add, sum_output, alpha, beta,
                 shortcut_activation, 0);
}

extern "C" void forward_convolutional_yolo_gpu(const float *input, const float *weights, const float *packed,
                                               const float *biases, const float *scales,
                                               const float *rolling_mean, const float *rolling_variance,
                                               float *output, int batch, int c, int h, int w, int n, int groups,
                                               int size, int stride, int pad, int batch_normalize, int activation,
                                               float *yolo_output, int n_anchors, int classes)
{
    if (!yolo_output) dn_fatal("forward_convolutional_yolo_gpu: null pointer");
    if (yolo_output == output) dn_fatal("forward_convolutional_yolo_gpu: yolo_output must not alias output");
    if (n_anchors <= 0 || classes < 0 || n != n_anchors * (5 + classes))
        dn_fatal("forward_convolutional_yolo_gpu: the filters must be n_anchors * (5 + classes)");
    conv_forward(input, weights, packed, biases, scales, rolling_mean, rolling_variance, output, batch, c, h, w,
                 n, groups, size, stride, pad, batch_normalize, activation, 0, yolo_output, 0.f, 0.f, DN_LINEAR,
                 5 + classes);
}

extern "C" int forward_convolutional_noalloc_gpu(const float *input, const float *weights, const float *packed,
                                                 const float *biases, const float *scales,
                                                 const float *rolling_mean, const float *rolling_variance,
                                                 float *output, int batch, int c, int h, int w, int n,
                                                 int groups, int size, int stride, int pad,
                                                 int batch_normalize, int activation)
{
    hip_require_device("forward_convolutional_noalloc_gpu");
    const int dev = hip_get_device();
    if (dev < 0 || dev >= DN_MAX_DEVICES) dn_fatal("forward_convolutional_noalloc_gpu: device index out of range");
    if (!g_scratch_dev[dev] || !g_cus_dev[dev]) conv_device_setup(); /* first call on this device */
    g_noalloc = 1;
    g_noalloc_error = 0;
    conv_forward(input, weights, packed, biases, scales, rolling_mean, rolling_variance, output, batch, c, h, w,
                 n, groups, size, stride, pad, batch_normalize, activation, 0, 0, 0.f, 0.f, DN_LINEAR, 0);
    g_noalloc = 0;
    if (g_noalloc_error) g_prof_start = g_prof_stop = 0; /* a pending timing pair must not stamp a later, unrelated call */
    return g_noalloc_error ? -1 : 0;
}

/* Whether forward_convolutional_maxpool_gpu serves the pair: a 3-channel 3x3 / stride 1 / pad 1
 * convolution of up to 64 filters with an activation its tail carries (leaky, linear, relu), over an
 * image of even height and a width that is a multiple of 32. */
extern "C" int conv_maxpool_fusable(int batch, int c, int h, int w, int n, int groups, int size, int stride, int pad,
                                    int activation)
{
    double slope;
    if (!conv_inline_activation(activation, &slope)) return 0;
    if (!conv_first_takes(c == 3 ? 3 : 13, c)) return 0;
    return conv_first_serves(batch, c, h, w, n, groups, size, stride, pad);
}

extern "C" void forward_convolutional_maxpool_gpu(const float *input, const float *weights, const float *biases,
                                                  const float *scales, const float *rolling_mean,
                                                  const float *rolling_variance, float *output, float *pool_output,
                                                  unsigned *next_xbits, int batch, int c, int h, int w, int n,
                                                  int groups, int size, int stride, int pad, int batch_normalize,
                                                  int activation)
{
    hip_require_device("forward_convolutional_maxpool_gpu");
    double slope = 1.;
    if (!input || !weights || !biases || !pool_output) dn_fatal("forward_convolutional_maxpool_gpu: null pointer");
    if (batch_normalize && (!scales || !rolling_mean || !rolling_variance))
        dn_fatal("forward_convolutional_maxpool_gpu: batch_normalize needs scales, rolling_mean, rolling_variance");
    if (!conv_maxpool_fusable(batch, c, h, w, n, groups, size, stride, pad, activation))
        dn_fatal("forward_convolutional_maxpool_gpu: serves 3x3 / 1 / pad 1 layers of 3 channels (up to 64 filters) or 16 "
                 "channels (up to 32) with a leaky, linear or relu activation, even height and a width that is a multiple "
                 "of 32, in the default fp32 mode (conv_maxpool_fusable)");
    conv_inline_activation(activation, &slope);
    const int dev = hip_get_device();
    if (dev < 0 || dev >= DN_MAX_DEVICES) dn_fatal("forward_convolutional_maxpool_gpu: device index out of range");
    if (!g_cus_dev[dev]) conv_device_setup();
    conv_first_forward(input, weights, biases, scales, rolling_mean, rolling_variance, output, pool_output, next_xbits,
                       batch, c, h, w, n, batch_normalize, slope, g_cus_dev[dev], 0, 0);
}
