/*
 * conv_first.hip - the first layer of an image network: 3 input channels, 3x3, stride 1, pad 1,
 * up to 64 filters (src/convolutional_layer.c:445-485 with c = 3), optionally together with the
 * 2x2 stride-2 maxpool behind it (src/maxpool_layer.c:79-114) and the sign bits an xnor
 * convolution behind that pool reads (src/convolutional_layer.c:43-49).
 *
 * With K = 27 the layer is neither a GEMM worth tiling (two K chunks) nor memory-bound in the
 * usual way: its 3-channel input is a 32nd of its output, and a kernel that re-derives weights,
 * batch-norm constants and index arithmetic per tile spends more issue cycles on that than on its
 * MFMAs (fp32 MFMA and the vector ALU share an issue port).  So:
 *
 *   - workgroups are persistent: each takes a contiguous run of tiles (XCD by XCD, so that tiles
 *     sharing input rows meet in one L2), loads its filters' weights into registers and computes the
 *     per-filter tail constants ONCE, and walks its run with the next tile's input already on its
 *     way to LDS while the current one is computed;
 *   - a tile is 256 pixels, a wave's share 2 rows x 32 columns; its shape is the widest of
 *     2 rows x 128 columns, 4 x 64 and 8 x 32 whose width divides the image's (416 = 13 x 32 takes the
 *     last: a 128-wide tile would leave a quarter of every fourth workgroup's waves idle).  Its input
 *     patch (rows + 2) x (columns + 8) x 3 channels, 4.8 to 6.4 KB, is copied by direct-to-LDS loads of
 *     16 bytes whose out-of-image quads come back as zeros from the buffer range check, so no tap
 *     needs a border test; the MFMA's pixel operand is one LDS read per (k pair, row) at a fixed offset;
 *   - K order is the reference's (channel, ky, kx), padded from 27 to 28; v_mfma_f32_32x32x2_f32 with
 *     the pixels as the row operand, so a lane owns one filter and, per row, four runs of four
 *     consecutive pixels: the 2x2 pooling window of the maxpool layer lies inside one lane;
 *   - outputs take a turn through LDS (16-byte quads XOR-swizzled by the filter) and leave in runs
 *     of a tile row per filter (512, 256 or 128 bytes); pooled outputs in runs of half that; the sign
 *     bits of the pooled map are one ballot per pooled pixel (lanes = filters = bits of the word).
 *
 * Results: the convolution's map is the same with and without the pooled outputs (one kernel, one
 * order of summation: k = 0..27 two at a time); the pooled map is the window-order maximum of those
 * values; the bits are (x > 0) of the pooled map.
 * When the map itself is not wanted (`out` null) the tail runs once per pooled pixel, on the
 * largest (for a negative batch-norm scale: the smallest) of the four sums - the tail is monotone
 * in its argument, rounding included, so the value is the same.
 */
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <float.h>
#include <stdint.h>

#include "device_math.h"
#include "hip.h"

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float float4u __attribute__((ext_vector_type(4), aligned(4)));

#define CF_THREADS 256
#define CF_PATCH_FLOATS 2048 /* two rounds of 256 lanes x 4 floats: the copy moves whole wave-loads */

/* Tile shapes, by WC = waves side by side in a tile row (4, 2, 1): */
#define CF_COLS(WC) (32 * (WC))                 /* columns of a tile */
#define CF_NRP(WC) (4 / (WC))                   /* row pairs of a tile */
#define CF_RS(WC) (CF_COLS(WC) + 8)             /* floats in a patch row: 4 halo + columns + 4 halo */
#define CF_PR(WC) (2 * CF_NRP(WC) + 2)          /* patch rows per channel */
#define CF_PATCH_QUADS(WC) (3 * CF_PR(WC) * (CF_RS(WC) / 4)) /* 408, 324, 300: at most 512 */

static inline hipStream_t dn_stream() { return (hipStream_t)hip_get_stream(); }

/* Workgroup barriers that leave vector-memory operations in flight: this wave's LDS traffic is done
 * (lgkmcnt), nothing is said about its global loads and stores.  __syncthreads() would wait for
 * those too - the direct-to-LDS load of the next tile's patch, the stores of the last tile - and
 * expose a trip to memory per barrier.  CF_BARRIER_ALL waits for everything (the first patch). */
#define CF_BARRIER() asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory")
#define CF_BARRIER_ALL() asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory")
/* s_waitcnt vmcnt(0) alone, as a builtin the compiler's own wait insertion sees (after it, it knows
 * of no load in flight and adds no waits of its own to the LDS accesses that follow):
 * simm16 = vmcnt[3:0] | expcnt(7) << 4 | lgkmcnt(15) << 8 | vmcnt[5:4] << 14 */
#define CF_WAIT_VM0() __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8))

struct first_args {
    const float *in;
    const float *w;                 /* [M][27] */
    const float *biases, *scales, *mean, *var;
    float *out;                     /* [B][M][H][W] or null */
    float *pool;                    /* [B][M][H/2][W/2] or null */
    unsigned *bits;                 /* [B][(M+31)/32][H/2][W/2] or null (needs pool) */
    int B, H, W, M, bn;
    int tiles_per_row, bands, ntiles; /* tiles across the image, bands of tile rows down it; B * bands * tiles_per_row */
    unsigned in_bytes;
    float slope_hi, slope_lo;
};

template <int TM, bool POOL, int WC>
__global__ __launch_bounds__(CF_THREADS, TM == 1 ? (POOL ? 3 : 4) : 2) void conv_first_kernel(first_args a)
{
    constexpr int C = CF_COLS(WC), NRP = CF_NRP(WC), RS = CF_RS(WC), PR = CF_PR(WC), QR = RS / 4;
    constexpr int R = 2 * NRP, PQ = CF_PATCH_QUADS(WC);
    typedef __attribute__((address_space(3))) void *lds_ptr;
    __shared__ __attribute__((aligned(16))) float patch0[CF_PATCH_FLOATS];
    __shared__ __attribute__((aligned(16))) float patch1[CF_PATCH_FLOATS];
    __shared__ __attribute__((aligned(16))) float stage[16 * 256];      /* 16 filters x the tile's 256 pixels */
    __shared__ __attribute__((aligned(16))) float pstage[POOL ? 32 * 64 : 4]; /* 32 filters x 64 pooled pixels */
    const int tid = threadIdx.x, lane = tid & 63, li = lane & 31, kh = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave / WC, wx = wave % WC; /* this wave's row pair and 32-column block of the tile */
    const int H = a.H, W = a.W, M = a.M, H2 = H >> 1, W2 = W >> 1;
    const dn_f2 slope = {a.slope_hi, a.slope_lo};

    /* this workgroup's run of tiles: XCD x (ids go round the eight XCDs) owns the x-th eighth of the
     * tile order, cut evenly among the workgroups that land on it */
    int t, t_end;
    {
        const int G = gridDim.x, xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
        const int gx = (G >> 3) + (xcd < (G & 7) ? 1 : 0); /* workgroups on this XCD */
        const int q = a.ntiles >> 3, r = a.ntiles & 7;
        const int x0 = xcd * q + (xcd < r ? xcd : r), nx = q + (xcd < r ? 1 : 0);
        t = x0 + (int)((long)nx * slot / gx);
        t_end = x0 + (int)((long)nx * (slot + 1) / gx);
    }
    if (t >= t_end) return;

    /* once per workgroup: this lane's filter(s) - weights of its k of every MFMA k pair, tail constants */
    float aw[TM][14];
    int koff[14];
    dn_tail_row row[TM];
#pragma unroll
    for (int s = 0; s < 14; ++s) {
        const int k = 2 * s + kh;
        const int ch = k / 9, r9 = k - 9 * ch, ky = r9 / 3, kx = r9 - 3 * ky;
        koff[s] = k < 27 ? (ch * PR + ky) * RS + kx + 3 : 0; /* pixel x sits in column x + 4 */
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int m = i * 32 + li;
            aw[i][s] = (k < 27 && m < M) ? a.w[m * 27 + k] : 0.f;
        }
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = i * 32 + li < M ? i * 32 + li : M - 1;
        row[i] = dn_tail_make(a.bn, a.biases[m], a.bn ? a.scales[m] : 1.f, a.bn ? a.mean[m] : 0.f,
                              a.bn ? a.var[m] : 1.f);
    }

    /* the two quads of the patch this lane copies, as (channel-row, quad of the row); fixed for all tiles */
    int q_cr[2], q_qx[2];
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        const int e = it * 256 + tid;
        q_cr[it] = e / QR;
        q_qx[it] = e - QR * q_cr[it];
    }
    const __amdgpu_buffer_rsrc_t in_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)a.in, 0, (int)a.in_bytes, 0x00020000);

    /* tile t = ((b * bands) + band) * tiles_per_row + cb */
    int cb = t % a.tiles_per_row, u = t / a.tiles_per_row;
    int rp = u % a.bands, b = u / a.bands; /* rp: the band */

    /* The LDS arrays reach the code below as __restrict__ parameters: once inlined, every access
     * carries the scope of its array, which is what lets the compiler tell a patch in flight (a
     * direct-to-LDS load counts in vmcnt) from the arrays being read and written; without it every
     * LDS access behind such a load would first wait for it. */
    auto load_patch = [&](float *__restrict__ buf, int lb, int lrp, int lcb) {
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int ch = q_cr[it] / PR, r = q_cr[it] - PR * ch;
            const int iy = R * lrp - 1 + r, xq = C * lcb + 4 * (q_qx[it] - 1);
            const bool ok = it * 256 + tid < PQ && (unsigned)iy < (unsigned)H && (unsigned)xq < (unsigned)W;
            const unsigned voff = ok ? (unsigned)((((lb * 3 + ch) * H + iy) * W + xq) * 4) : 0xFFFFFFF0u;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(in_rsrc, (lds_ptr)&buf[(it * 256 + wave * 64) * 4], 16, voff, 0, 0, 0);
        }
    };

    load_patch(patch0, b, rp, cb);
    /* one tile: `buf` holds its patch, `nbuf` receives the next tile's */
    auto do_tile = [&](const float *__restrict__ buf, float *__restrict__ nbuf, float *__restrict__ stg,
                       float *__restrict__ pstg) {
        /* next tile's coordinates */
        int ncb = cb + 1, nrp = rp, nb = b;
        if (ncb == a.tiles_per_row) {
            ncb = 0;
            if (++nrp == a.bands) {
                nrp = 0;
                ++nb;
            }
        }
        /* On entry this tile's patch is in `buf` and visible to every wave, and every wave is through
         * with `nbuf`.  This barrier only says that the staging buffers' last readers are done. */
        CF_BARRIER();
        const int x0 = C * cb;
        const int tc = W - x0 < C ? W - x0 : C; /* columns of this tile: a multiple of 32 (short only when WC = 4) */
        const bool active = 32 * wx < tc;       /* wave-uniform */

        f32x16 acc[TM][2];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
        if (active) {
            const int base = 2 * wr * RS + 32 * wx + li;
#pragma unroll
            for (int s = 0; s < 14; ++s) {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const float bv = buf[base + j * RS + koff[s]];
#pragma unroll
                    for (int i = 0; i < TM; ++i)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv, aw[i][s], acc[i][j], 0, 0, 0);
                }
            }
        }

        /* The next tile's patch is requested now that this one has been read, and waited for once,
         * below, in front of this tile's first store: by then it has had the tail arithmetic's time, and
         * the previous tile's stores a whole tile.  (Waiting anywhere behind this tile's stores would
         * wait for them too: a trip to memory per tile.) */
        if (t + 1 < t_end) load_patch(nbuf, nb, nrp, ncb);

        /* acc[i][j][4g + q]: filter 32i + li, row R band + 2wr + j, column x0 + 32wx + 8g + 4kh + q */
        float pooled[TM][8];
        if (a.out) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[i][j][r] = dn_tail(acc[i][j][r], row[i], slope);
            if (POOL) {
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int g = 0; g < 4; ++g)
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            float m = -FLT_MAX; /* the window in the pooling layer's order: first maximum wins */
                            if (acc[i][0][4 * g + 2 * h] > m) m = acc[i][0][4 * g + 2 * h];
                            if (acc[i][0][4 * g + 2 * h + 1] > m) m = acc[i][0][4 * g + 2 * h + 1];
                            if (acc[i][1][4 * g + 2 * h] > m) m = acc[i][1][4 * g + 2 * h];
                            if (acc[i][1][4 * g + 2 * h + 1] > m) m = acc[i][1][4 * g + 2 * h + 1];
                            pooled[i][2 * g + h] = m;
                        }
            }
        }
        CF_WAIT_VM0(); /* the next patch has landed (every path comes by here); the next barrier publishes it */
        if (a.out) {
            /* the map, 16 filters at a time through LDS */
#pragma unroll
            for (int i = 0; i < TM; ++i) {
#pragma unroll
                for (int hf = 0; hf < 2; ++hf) {
                    if (i + hf > 0) CF_BARRIER(); /* the rows stored last have been read */
                    if (active && (li >> 4) == hf) {
                        const int f16 = li & 15;
#pragma unroll
                        for (int j = 0; j < 2; ++j)
#pragma unroll
                            for (int g = 0; g < 4; ++g) {
                                const int qd = (2 * wr + j) * (8 * WC) + 8 * wx + 2 * g + kh; /* quad of the tile */
                                float4 o;
                                o.x = acc[i][j][4 * g + 0];
                                o.y = acc[i][j][4 * g + 1];
                                o.z = acc[i][j][4 * g + 2];
                                o.w = acc[i][j][4 * g + 3];
                                *(float4 *)&stg[(f16 * 64 + (qd ^ f16)) * 4] = o;
                            }
                    }
                    CF_BARRIER();
#pragma unroll
                    for (int it = 0; it < 4; ++it) {
                        const int id = it * 256 + tid;
                        const int f16 = id >> 6, qd = id & 63, j = qd / (8 * WC), q = qd % (8 * WC);
                        const int m = i * 32 + hf * 16 + f16;
                        if (4 * q < tc && m < M) {
                            const float4 o = *(const float4 *)&stg[(f16 * 64 + (qd ^ f16)) * 4];
                            *(float4u *)(a.out + (((long)b * M + m) * H + R * rp + j) * W + x0 + 4 * q) =
                                (float4u){o.x, o.y, o.z, o.w};
                        }
                    }
                }
            }
        } else if (POOL) {
            /* the map is not wanted: the tail once per pooled pixel, on the sum it is largest for */
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const float s0 = acc[i][0][4 * g + 2 * h], s1 = acc[i][0][4 * g + 2 * h + 1];
                        const float s2 = acc[i][1][4 * g + 2 * h], s3 = acc[i][1][4 * g + 2 * h + 1];
                        const float hi = fmaxf(fmaxf(s0, s1), fmaxf(s2, s3)), lo = fminf(fminf(s0, s1), fminf(s2, s3));
                        const float v = dn_tail(row[i].scale >= 0.f ? hi : lo, row[i], slope);
                        pooled[i][2 * g + h] = v > -FLT_MAX ? v : -FLT_MAX;
                    }
        }

        if (POOL) {
            const int PW = W2, px0 = x0 >> 1, pc = tc >> 1; /* pooled columns of this tile */
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                if (i > 0) CF_BARRIER();
                if (active) {
                    /* pooled[i][2g + h]: filter 32i + li, pooled row NRP band + wr, column px0 + 16wx + 4g + 2kh + h */
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int p2 = wr * (8 * WC) + 8 * wx + 2 * g + kh; /* pair of the tile's 64 pooled pixels */
                        *(float2 *)&pstg[(li * 32 + (p2 ^ ((li & 15) << 1))) * 2] =
                            make_float2(pooled[i][2 * g], pooled[i][2 * g + 1]);
                    }
                    if (a.bits) {
                        /* one ballot per pooled pixel pair: the lanes of a half-wave are the 32 filters of the word */
                        unsigned word = 0;
#pragma unroll
                        for (int g = 0; g < 4; ++g)
#pragma unroll
                            for (int h = 0; h < 2; ++h) {
                                const unsigned long long m64 = __ballot(pooled[i][2 * g + h] > 0.f);
                                /* lane tt < 16 keeps the word of pooled column 16wx + tt, tt = 4g + 2kh' + h */
                                if (lane == 4 * g + h) word = (unsigned)m64;
                                if (lane == 4 * g + 2 + h) word = (unsigned)(m64 >> 32);
                            }
                        const int valid = M - 32 * i; /* filters of this word */
                        if (valid < 32) word &= (1u << valid) - 1u;
                        if (lane < 16) {
                            const int cwn = (M + 31) >> 5;
                            a.bits[(((long)b * cwn + i) * H2 + NRP * rp + wr) * PW + px0 + 16 * wx + lane] = word;
                        }
                    }
                }
                CF_BARRIER();
#pragma unroll
                for (int it = 0; it < 2; ++it) {
                    const int id = it * 256 + tid;
                    const int f = id >> 4, qq = id & 15, pj = qq / (4 * WC), pq = qq % (4 * WC);
                    const int m = i * 32 + f;
                    if (4 * pq < pc && m < M) {
                        const float4 o = *(const float4 *)&pstg[(f * 16 + (qq ^ (f & 15))) * 4];
                        *(float4u *)(a.pool + (((long)b * M + m) * H2 + NRP * rp + pj) * PW + px0 + 4 * pq) =
                            (float4u){o.x, o.y, o.z, o.w};
                    }
                }
            }
        }
        cb = ncb;
        rp = nrp;
        b = nb;
    };
    __builtin_amdgcn_s_waitcnt(0); /* the first patch */
    CF_BARRIER();
    for (;;) {
        do_tile(patch0, patch1, stage, pstage);
        if (++t >= t_end) break;
        do_tile(patch1, patch0, stage, pstage);
        if (++t >= t_end) break;
    }
    __builtin_amdgcn_s_waitcnt(0); /* no wave ends with a direct-to-LDS load in flight */
}

/* Whether conv_first_kernel serves the layer (then also with the pooled outputs). */
extern "C" int conv_first_serves(int batch, int c, int h, int w, int n, int groups, int size, int stride, int pad)
{
    if (groups != 1 || c != 3 || size != 3 || stride != 1 || pad != 1 || n < 1 || n > 64) return 0;
    if (batch < 1 || h < 2 || (h & 1) || w < 32 || (w & 31)) return 0;
    if ((long)batch * 3 * h * w * 4 >= (1L << 32) - 64) return 0; /* 32-bit buffer offsets */
    if ((long)batch * (h / 2) * (w / 32) >= (1L << 31)) return 0;
    return 1;
}

/* The tile shape, as waves side by side: the widest tile whose width divides the image's and whose
 * height divides its height; failing all, the 128-wide tile with a short last column of tiles.
 * g_shape != 0 forces a shape where the image allows it (tests, sweeps). */
static int g_shape = 0;

extern "C" void conv_first_set_shape(int waves_across) { g_shape = waves_across; }

static int shape_fits(int wc, int h, int w) { return w % (32 * wc) == 0 && h % (2 * (4 / wc)) == 0; }

static int pick_shape(int h, int w)
{
    if ((g_shape == 4 || g_shape == 2 || g_shape == 1) && (g_shape == 4 || shape_fits(g_shape, h, w))) return g_shape;
    if (shape_fits(4, h, w)) return 4;
    if (shape_fits(2, h, w)) return 2;
    if (shape_fits(1, h, w)) return 1;
    return 4;
}

template <int TM, bool POOL>
static const void *kernel_of_shape(int wc)
{
    return wc == 4 ? (const void *)conv_first_kernel<TM, POOL, 4>
         : wc == 2 ? (const void *)conv_first_kernel<TM, POOL, 2>
                   : (const void *)conv_first_kernel<TM, POOL, 1>;
}

extern "C" const char *conv_first_kernel_name(int n, int pooled, int h, int w)
{
    static const char *const names[2][2][3] = {
        {{"conv_first_kernel<1,false,1>", "conv_first_kernel<1,false,2>", "conv_first_kernel<1,false,4>"},
         {"conv_first_kernel<1,true,1>", "conv_first_kernel<1,true,2>", "conv_first_kernel<1,true,4>"}},
        {{"conv_first_kernel<2,false,1>", "conv_first_kernel<2,false,2>", "conv_first_kernel<2,false,4>"},
         {"conv_first_kernel<2,true,1>", "conv_first_kernel<2,true,2>", "conv_first_kernel<2,true,4>"}}};
    const int wc = pick_shape(h, w);
    return names[n > 32][pooled != 0][wc >> 1];
}

/* The launch.  `out` or `pool` may be null (not both); `bits` needs `pool`.  slope: the activation as
 * y > 0 ? y : slope*y.  start/stop: events to attach to the dispatch, or null. */
extern "C" void conv_first_forward(const float *input, const float *weights, const float *biases, const float *scales,
                                   const float *rolling_mean, const float *rolling_variance, float *out, float *pool,
                                   unsigned *bits, int batch, int h, int w, int n, int batch_normalize, double slope,
                                   int cus, void *start, void *stop)
{
    if (!conv_first_serves(batch, 3, h, w, n, 1, 3, 1, 1)) dn_fatal("conv_first_forward: geometry not served");
    if ((!out && !pool) || (bits && !pool)) dn_fatal("conv_first_forward: nothing to write");
    const int wc = pick_shape(h, w);
    first_args a;
    a.in = input;
    a.w = weights;
    a.biases = biases;
    a.scales = scales;
    a.mean = rolling_mean;
    a.var = rolling_variance;
    a.out = out;
    a.pool = pool;
    a.bits = bits;
    a.B = batch;
    a.H = h;
    a.W = w;
    a.M = n;
    a.bn = batch_normalize ? 1 : 0;
    a.tiles_per_row = (w + 32 * wc - 1) / (32 * wc);
    a.bands = h / (2 * (4 / wc));
    if (a.bands * 2 * (4 / wc) != h) dn_fatal("conv_first_forward: tile shape does not divide the image");
    a.ntiles = batch * a.bands * a.tiles_per_row;
    a.in_bytes = (unsigned)((long)batch * 3 * h * w * 4);
    const dn_f2 s = dn_split(slope);
    a.slope_hi = s.hi;
    a.slope_lo = s.lo;
    const void *kernel = pool ? (n <= 32 ? kernel_of_shape<1, true>(wc) : kernel_of_shape<2, true>(wc))
                              : (n <= 32 ? kernel_of_shape<1, false>(wc) : kernel_of_shape<2, false>(wc));
    /* exactly as many workgroups as stay resident (two to four per CU, by the variant's registers), each
     * walking its run: one more per CU would start when the others end and run alone */
    static int resident[2][2][3];
    int *per_cu = &resident[n > 32][pool != 0][wc >> 1];
    if (!*per_cu) {
        int nb = 0;
        hip_check_error(hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, kernel, CF_THREADS, 0));
        *per_cu = nb < 1 ? 1 : nb > 4 ? 4 : nb;
    }
    long grid = (long)(cus > 0 ? cus : 256) * *per_cu;
    if (grid > a.ntiles) grid = a.ntiles;
    void *args[] = {&a};
    if (start)
        hip_check_error(hipExtLaunchKernel(kernel, dim3((unsigned)grid), dim3(CF_THREADS), args, 0, dn_stream(),
                                           (hipEvent_t)start, (hipEvent_t)stop, 0));
    else
        hip_check_error(hipLaunchKernel(kernel, dim3((unsigned)grid), dim3(CF_THREADS), args, 0, dn_stream()));
    dn_check_launch("conv_first_forward");
}
