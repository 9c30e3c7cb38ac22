/*
 * conv_first.hip - the first layers of an image network: 3x3, stride 1, pad 1 over 3 input channels
 * (up to 64 filters) or over the 16 channels behind a pooled first layer (up to 32 filters)
 * (src/convolutional_layer.c:445-485), optionally together with the 2x2 stride-2 maxpool behind the
 * layer (src/maxpool_layer.c:79-114) and the sign bits an xnor convolution behind that pool reads
 * (src/convolutional_layer.c:43-49).
 *
 * With K = 27 (or 144) the layer is neither a GEMM worth tiling (two to nine K chunks) nor
 * memory-bound in the usual way: its output is many times its input, and a kernel that re-derives
 * weights, batch-norm constants and index arithmetic per tile spends more issue cycles on that than
 * on its MFMAs (fp32 MFMA and the vector ALU share an issue port).  So:
 *
 *   - workgroups are persistent: each takes a contiguous run of tiles (XCD by XCD, so that tiles
 *     sharing input rows meet in one L2), loads its filters' weights into registers and computes the
 *     per-filter tail constants ONCE, and walks its run with the next tile's input already on its
 *     way to LDS while the current one is computed;
 *   - a tile is 256 pixels, a wave's share 2 rows x 32 columns; its shape is 2 rows x 128 columns,
 *     4 x 64 or 8 x 32, whichever wastes the fewest columns in the last tile of a row (416 = 13 x 32
 *     and 208 = 6.5 x 32 take the last).  Its input patch, (rows + 2) x (columns + 8) per channel, is
 *     copied by direct-to-LDS loads of 16 bytes whose out-of-image quads come back as zeros from
 *     the buffer range check, so no tap needs a border test; the MFMA's pixel operand is one LDS
 *     read per (k pair, row) at a fixed offset;
 *   - v_mfma_f32_32x32x2_f32 with the pixels as the row operand, so a lane owns one filter and, per
 *     row, four runs of four consecutive pixels: the 2x2 pooling window of the maxpool layer lies
 *     inside one lane.  K order: 3 channels - the reference's (channel, ky, kx), padded from 27 to 28,
 *     two at a time; 16 channels - tap by tap over the channel pairs (ch, ch + 8), which makes every
 *     LDS offset of the loop an immediate;
 *   - outputs take a turn through LDS (16-byte quads XOR-swizzled by the filter) and leave in runs
 *     of a tile row per filter (512, 256 or 128 bytes); pooled outputs in runs of half that; the sign
 *     bits of the pooled map are one ballot per pooled pixel (lanes = filters = bits of the word).
 *
 * Results: the convolution's map is the same with and without the pooled outputs and whatever the
 * tile shape (one kernel, one order of summation); the pooled map is the window-order maximum of those
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
/* Tile shapes, by WC = waves side by side in a tile row (4, 2, 1): */
#define CF_COLS(WC) (32 * (WC))                 /* columns of a tile */
#define CF_NRP(WC) (4 / (WC))                   /* row pairs of a tile */
#define CF_RS(WC) (CF_COLS(WC) + 8)             /* floats in a patch row: 4 halo + columns + 4 halo */
#define CF_PR(WC) (2 * CF_NRP(WC) + 2)          /* patch rows per channel */
#define CF_PATCH_QUADS(WC, C) ((C) * CF_PR(WC) * (CF_RS(WC) / 4)) /* 3 channels: 408, 324, 300; 16: 2176, 1728, 1600 */
#define CF_ROUNDS(WC, C) ((CF_PATCH_QUADS(WC, C) + 255) / 256)   /* the copy moves whole wave-loads: 256 lanes x 16 bytes */

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

/* LDS reads the compiler does not see.  The 16-channel loop reads its patch while the next tile's
 * patch is on its way into the other buffer; an LDS read the compiler knows of would first wait for
 * that direct-to-LDS load whenever it cannot prove the two buffers apart (it can for one of the two
 * unrolled tile instances, not for the other), and the wait is the whole trip to memory.  So these
 * reads are written out: ds_read_b32 with an immediate offset from one address register, and one
 * s_waitcnt lgkmcnt(0) that the values pass through (as in-out operands) before their first use.
 * What makes them safe is what the kernel does anyway: a patch is only read in the tile after the one
 * that waited for its load (vmcnt 0) and crossed a workgroup barrier. */
template <int OFF>
__device__ __forceinline__ float cf_lds_read(unsigned addr)
{
    float v;
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
    return v;
}

/* the 4 x 3 patch values of channel CH that the 18 MFMAs of a lane's two output rows use: v[3 r + kx] */
template <int PR, int RS, int CH, int I = 0>
__device__ __forceinline__ void cf_read_channel(float (&v)[12], unsigned addr)
{
    if constexpr (I < 12) {
        v[I] = cf_lds_read<((CH * PR + I / 3) * RS + I % 3 + 3) * 4>(addr);
        cf_read_channel<PR, RS, CH, I + 1>(v, addr);
    }
}

__device__ __forceinline__ void cf_wait_lds(float (&v)[12])
{
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]),
                   "+v"(v[8]), "+v"(v[9]), "+v"(v[10]), "+v"(v[11]));
}

/* Channels CH .. HALF-1 of the 16-channel loop: channel CH's values are in `cur`; the next channel's
 * are requested in front of this channel's MFMAs and waited for behind them. */
template <int TM, int PR, int RS, int HALF, int NS, int CH = 0>
__device__ __forceinline__ void cf_channels(f32x16 (&acc)[TM][2], const float (&aw)[TM][NS], float (&cur)[12], unsigned addr)
{
    if constexpr (CH < HALF) {
        float nxt[12];
        if constexpr (CH + 1 < HALF) cf_read_channel<PR, RS, CH + 1>(nxt, addr);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ky = 0; ky < 3; ++ky)
#pragma unroll
            for (int kx = 0; kx < 3; ++kx)
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int i = 0; i < TM; ++i)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(cur[(ky + j) * 3 + kx], aw[i][CH * 9 + ky * 3 + kx],
                                                                         acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (CH + 1 < HALF) {
            cf_wait_lds(nxt);
            cf_channels<TM, PR, RS, HALF, NS, CH + 1>(acc, aw, nxt, addr);
        }
    }
}

struct first_args {
    const float *in;
    const float *w;                 /* [M][9 C] */
    const float *biases, *scales, *mean, *var;
    float *out;                     /* [B][M][H][W] or null */
    float *pool;                    /* [B][M][H/2][W/2] or null */
    unsigned *bits;                 /* [B][(M+31)/32][H/2][W/2] or null (needs pool) */
    int B, H, W, M, bn;
    int tiles_per_row, bands, ntiles; /* tiles across the image, bands of tile rows down it; B * bands * tiles_per_row */
    unsigned in_bytes;
    float slope_hi, slope_lo;
};

template <int TM, bool POOL, int WC, int C>
__global__ __launch_bounds__(CF_THREADS, C > 3 ? 2 : TM == 1 ? (POOL ? 3 : 4) : 2) void conv_first_kernel(first_args a)
{
    constexpr int COLS = CF_COLS(WC), NRP = CF_NRP(WC), RS = CF_RS(WC), PR = CF_PR(WC), QR = RS / 4;
    constexpr int R = 2 * NRP, PQ = CF_PATCH_QUADS(WC, C), ROUNDS = CF_ROUNDS(WC, C);
    constexpr int K = 9 * C, NS = (K + 1) / 2; /* MFMA k pairs */
    /* Which two k a pair holds.  3 channels: k = 2s + kh, the reference's order two at a time.  An even
     * number of channels: k = s + NS kh, i.e. the same tap of channel ch and of channel ch + C/2 - the
     * second k's LDS offset is then the first's plus a constant, and every offset of the MFMA loop
     * is an immediate instead of a register. */
    constexpr bool SPLIT_CH = (C % 2) == 0;
    typedef __attribute__((address_space(3))) void *lds_ptr;
    __shared__ __attribute__((aligned(16))) float patch0[ROUNDS * 1024];
    __shared__ __attribute__((aligned(16))) float patch1[ROUNDS * 1024];
    /* 16 filters x the tile's 256 pixels; the pooled map (32 filters x 64 pooled pixels) takes its turn
     * through the same buffer afterwards */
    __shared__ __attribute__((aligned(16))) float stage[16 * 256];
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
    float aw[TM][NS];
    int koff[SPLIT_CH ? 1 : NS]; /* 3 channels: LDS offset of this lane's k of pair s */
    dn_tail_row row[TM];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        const int k = SPLIT_CH ? s + NS * kh : 2 * s + kh;
        if constexpr (!SPLIT_CH) {
            const int ch = k / 9, r9 = k - 9 * ch, ky = r9 / 3, kx = r9 - 3 * ky;
            koff[s] = k < K ? (ch * PR + ky) * RS + kx + 3 : 0; /* pixel x sits in column x + 4 */
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int m = i * 32 + li;
            aw[i][s] = (k < K && m < M) ? a.w[m * K + k] : 0.f;
        }
    }
    const int khoff = SPLIT_CH ? kh * (C / 2) * PR * RS : 0;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = i * 32 + li < M ? i * 32 + li : M - 1;
        row[i] = dn_tail_make(a.bn, a.biases[m], a.bn ? a.scales[m] : 1.f, a.bn ? a.mean[m] : 0.f,
                              a.bn ? a.var[m] : 1.f);
    }

    /* the quads of the patch this lane copies (one per round of 256 lanes), fixed for all tiles: byte
     * offset relative to the tile's first patch element, and (patch row, quad of the row) for the
     * border tests */
    int q_rel[ROUNDS], q_rq[ROUNDS];
#pragma unroll
    for (int it = 0; it < ROUNDS; ++it) {
        const int e = it * 256 + tid;
        const int cr = e / QR, qx = e - QR * cr, ch = cr / PR, r = cr - PR * ch;
        q_rel[it] = e < PQ ? ((ch * H + r) * W + 4 * qx) * 4 : -1;
        q_rq[it] = r | (qx << 8);
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
        const int y_top = R * lrp - 1, x_left = COLS * lcb - 4; /* image coordinates of the patch's first element */
        /* modulo 2^32: the origin may lie above or left of the tensor, the sum with a valid quad's offset does not */
        const unsigned origin = (((unsigned)(lb * C * H) + (unsigned)y_top) * (unsigned)W + (unsigned)x_left) * 4u;
#pragma unroll
        for (int it = 0; it < ROUNDS; ++it) {
            const int iy = y_top + (q_rq[it] & 255), xq = x_left + 4 * (q_rq[it] >> 8);
            const bool ok = q_rel[it] >= 0 && (unsigned)iy < (unsigned)H && (unsigned)xq < (unsigned)W;
            const unsigned voff = ok ? origin + (unsigned)q_rel[it] : 0xFFFFFFF0u;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(in_rsrc, (lds_ptr)&buf[(it * 256 + wave * 64) * 4], 16, voff, 0, 0, 0);
        }
    };

    load_patch(patch0, b, rp, cb);
    /* one tile: `buf` holds its patch, `nbuf` receives the next tile's */
    auto do_tile = [&](const float *__restrict__ buf, float *__restrict__ nbuf, float *__restrict__ stg) {
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
        const int x0 = COLS * cb;
        const int tc = W - x0 < COLS ? W - x0 : COLS; /* columns of this tile: a multiple of 8 (the last of a row may be short) */
        const bool active = 32 * wx < tc;       /* wave-uniform */

        /* 16 channels: the next tile's patch (25 KB and more) is requested in front of this tile's 144
         * MFMAs, which give it four microseconds to land; with 3 channels the MFMAs are too few to
         * matter and the request follows them (below) */
        if (C > 3 && t + 1 < t_end) load_patch(nbuf, nb, nrp, ncb);

        f32x16 acc[TM][2];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
        if (active) {
            const int base = 2 * wr * RS + 32 * wx + li + khoff;
            if constexpr (SPLIT_CH) {
                /* Pair s = 9 ch + 3 ky + kx is tap (ky, kx) of channel ch (and of channel ch + C/2 in the
                 * other half-wave).  The two output rows of a wave share patch rows (row j, tap row ky
                 * reads patch row ky + j), so a channel needs 4 x 3 values for its 18 MFMAs; they are read
                 * one channel ahead (cf_channels). */
                typedef __attribute__((address_space(3))) float lds_float;
                const unsigned addr = (unsigned)(unsigned long)(const lds_float *)buf + 4u * (unsigned)base;
                float cur[12];
                cf_read_channel<PR, RS, 0>(cur, addr);
                cf_wait_lds(cur);
                cf_channels<TM, PR, RS, C / 2, NS>(acc, aw, cur, addr);
            } else {
#pragma unroll
                for (int s = 0; s < NS; ++s) {
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        const float bv = buf[base + j * RS + koff[s]];
#pragma unroll
                        for (int i = 0; i < TM; ++i)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv, aw[i][s], acc[i][j], 0, 0, 0);
                    }
                }
            }
        }

        /* The next tile's patch is requested now that this one has been read, and waited for once,
         * below, in front of this tile's first store: by then it has had the tail arithmetic's time, and
         * the previous tile's stores a whole tile.  (Waiting anywhere behind this tile's stores would
         * wait for them too: a trip to memory per tile.) */
        if (C == 3 && t + 1 < t_end) load_patch(nbuf, nb, nrp, ncb);

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
            float *__restrict__ pstg = stg;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                if (i > 0 || a.out) CF_BARRIER(); /* the buffer's last readers (the map's rows, the pooled rows before) are done */
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
                        if (lane < 16 && 16 * wx + lane < pc) { /* a short last tile holds fewer pooled columns */
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
        do_tile(patch0, patch1, stage);
        if (++t >= t_end) break;
        do_tile(patch1, patch0, stage);
        if (++t >= t_end) break;
    }
    __builtin_amdgcn_s_waitcnt(0); /* no wave ends with a direct-to-LDS load in flight */
}

/* ---- up to 16 filters over 3 channels (the first layer of the tiny networks) ----------------------
 * The same workgroup, tile, patch and staging scheme on v_mfma_f32_16x16x4_f32: with 16 filters or
 * fewer the 32x32 MFMA multiplies sixteen rows of zeros and the tail runs on them too.  Here the
 * pixels are again the row operand: lane (p = lane % 16, g = lane / 16) feeds pixel p and k = 4s + g
 * of MFMA s (seven of them for K = 27, padded to 28), and owns filter lane % 16 at pixels 4g .. 4g+3
 * of each 16-pixel block - a wave's 2 rows x 32 columns are four blocks (row j, half h), sixteen
 * outputs per lane instead of thirty-two.  The 2x2 pooling window still lies inside one lane; a
 * ballot's 64 bits are four 16-filter words (one per g). */
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <bool POOL, int WC>
__global__ __launch_bounds__(CF_THREADS, 4) void conv_first16_kernel(first_args a)
{
    constexpr int C = 3, COLS = CF_COLS(WC), NRP = CF_NRP(WC), RS = CF_RS(WC), PR = CF_PR(WC), QR = RS / 4;
    constexpr int R = 2 * NRP, PQ = CF_PATCH_QUADS(WC, C), ROUNDS = CF_ROUNDS(WC, C);
    constexpr int K = 27, NS = 7; /* MFMA k quads */
    typedef __attribute__((address_space(3))) void *lds_ptr;
    __shared__ __attribute__((aligned(16))) float patch0[ROUNDS * 1024];
    __shared__ __attribute__((aligned(16))) float patch1[ROUNDS * 1024];
    __shared__ __attribute__((aligned(16))) float stage[16 * 256]; /* 16 filters x the tile's 256 pixels, then the pooled map */
    const int tid = threadIdx.x, lane = tid & 63, f = lane & 15, g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave / WC, wx = wave % WC;
    const int H = a.H, W = a.W, M = a.M, H2 = H >> 1, W2 = W >> 1;
    const dn_f2 slope = {a.slope_hi, a.slope_lo};

    int t, t_end;
    {
        const int G = gridDim.x, xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
        const int gx = (G >> 3) + (xcd < (G & 7) ? 1 : 0);
        const int q = a.ntiles >> 3, r = a.ntiles & 7;
        const int x0 = xcd * q + (xcd < r ? xcd : r), nx = q + (xcd < r ? 1 : 0);
        t = x0 + (int)((long)nx * slot / gx);
        t_end = x0 + (int)((long)nx * (slot + 1) / gx);
    }
    if (t >= t_end) return;

    /* once per workgroup: this lane's filter - the weight of its k of every MFMA, the tail constants */
    float aw[NS];
    int koff[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        const int k = 4 * s + g;
        const int ch = k / 9, r9 = k - 9 * ch, ky = r9 / 3, kx = r9 - 3 * ky;
        koff[s] = k < K ? (ch * PR + ky) * RS + kx + 3 : 0; /* pixel x sits in column x + 4 */
        aw[s] = (k < K && f < M) ? a.w[f * K + k] : 0.f;
    }
    const int mf = f < M ? f : M - 1;
    const dn_tail_row row = dn_tail_make(a.bn, a.biases[mf], a.bn ? a.scales[mf] : 1.f, a.bn ? a.mean[mf] : 0.f,
                                         a.bn ? a.var[mf] : 1.f);

    int q_rel[ROUNDS], q_rq[ROUNDS];
#pragma unroll
    for (int it = 0; it < ROUNDS; ++it) {
        const int e = it * 256 + tid;
        const int cr = e / QR, qx = e - QR * cr, ch = cr / PR, r = cr - PR * ch;
        q_rel[it] = e < PQ ? ((ch * H + r) * W + 4 * qx) * 4 : -1;
        q_rq[it] = r | (qx << 8);
    }
    const __amdgpu_buffer_rsrc_t in_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)a.in, 0, (int)a.in_bytes, 0x00020000);

    int cb = t % a.tiles_per_row, u = t / a.tiles_per_row;
    int rp = u % a.bands, b = u / a.bands; /* rp: the band */

    auto load_patch = [&](float *__restrict__ buf, int lb, int lrp, int lcb) {
        const int y_top = R * lrp - 1, x_left = COLS * lcb - 4;
        const unsigned origin = (((unsigned)(lb * C * H) + (unsigned)y_top) * (unsigned)W + (unsigned)x_left) * 4u;
#pragma unroll
        for (int it = 0; it < ROUNDS; ++it) {
            const int iy = y_top + (q_rq[it] & 255), xq = x_left + 4 * (q_rq[it] >> 8);
            const bool ok = q_rel[it] >= 0 && (unsigned)iy < (unsigned)H && (unsigned)xq < (unsigned)W;
            const unsigned voff = ok ? origin + (unsigned)q_rel[it] : 0xFFFFFFF0u;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(in_rsrc, (lds_ptr)&buf[(it * 256 + wave * 64) * 4], 16, voff, 0, 0, 0);
        }
    };

    load_patch(patch0, b, rp, cb);
    auto do_tile = [&](const float *__restrict__ buf, float *__restrict__ nbuf, float *__restrict__ stg) {
        int ncb = cb + 1, nrp = rp, nb = b;
        if (ncb == a.tiles_per_row) {
            ncb = 0;
            if (++nrp == a.bands) {
                nrp = 0;
                ++nb;
            }
        }
        CF_BARRIER(); /* the staging buffer's last readers are done */
        const int x0 = COLS * cb;
        const int tc = W - x0 < COLS ? W - x0 : COLS;
        const bool active = 32 * wx < tc; /* wave-uniform */

        f32x4 acc[2][2]; /* [row j][16-column half h]: filter f, columns x0 + 32wx + 16h + 4g + (0..3) */
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int h = 0; h < 2; ++h) acc[j][h] = (f32x4){0.f, 0.f, 0.f, 0.f};
        if (active) {
            const int base = 2 * wr * RS + 32 * wx + f; /* as the pixel operand, lane % 16 is the pixel of the block */
#pragma unroll
            for (int s = 0; s < NS; ++s)
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int h = 0; h < 2; ++h)
                        acc[j][h] = __builtin_amdgcn_mfma_f32_16x16x4f32(buf[base + j * RS + 16 * h + koff[s]], aw[s],
                                                                         acc[j][h], 0, 0, 0);
        }
        if (t + 1 < t_end) load_patch(nbuf, nb, nrp, ncb);

        float pooled[2][2]; /* [half h][e]: pooled column 8h + 2g + e of the wave's sixteen */
        if (a.out) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[j][h][r] = dn_tail(acc[j][h][r], row, slope);
            if (POOL) {
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int e = 0; e < 2; ++e) {
                        float m = -FLT_MAX; /* the window in the pooling layer's order: first maximum wins */
                        if (acc[0][h][2 * e] > m) m = acc[0][h][2 * e];
                        if (acc[0][h][2 * e + 1] > m) m = acc[0][h][2 * e + 1];
                        if (acc[1][h][2 * e] > m) m = acc[1][h][2 * e];
                        if (acc[1][h][2 * e + 1] > m) m = acc[1][h][2 * e + 1];
                        pooled[h][e] = m;
                    }
            }
        }
        CF_WAIT_VM0(); /* the next patch has landed (every path comes by here); the next barrier publishes it */
        if (a.out) {
            if (active) {
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const int qd = (2 * wr + j) * (8 * WC) + 8 * wx + 4 * h + g; /* quad of the tile */
                        float4 o;
                        o.x = acc[j][h][0];
                        o.y = acc[j][h][1];
                        o.z = acc[j][h][2];
                        o.w = acc[j][h][3];
                        *(float4 *)&stg[(f * 64 + (qd ^ f)) * 4] = o;
                    }
            }
            CF_BARRIER();
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                const int id = it * 256 + tid;
                const int m = id >> 6, qd = id & 63, j = qd / (8 * WC), q = qd % (8 * WC);
                if (4 * q < tc && m < M) {
                    const float4 o = *(const float4 *)&stg[(m * 64 + (qd ^ m)) * 4];
                    *(float4u *)(a.out + (((long)b * M + m) * H + R * rp + j) * W + x0 + 4 * q) =
                        (float4u){o.x, o.y, o.z, o.w};
                }
            }
        } else if (POOL) {
            /* the map is not wanted: the tail once per pooled pixel, on the sum it is largest for */
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const float s0 = acc[0][h][2 * e], s1 = acc[0][h][2 * e + 1];
                    const float s2 = acc[1][h][2 * e], s3 = acc[1][h][2 * e + 1];
                    const float hi = fmaxf(fmaxf(s0, s1), fmaxf(s2, s3)), lo = fminf(fminf(s0, s1), fminf(s2, s3));
                    const float v = dn_tail(row.scale >= 0.f ? hi : lo, row, slope);
                    pooled[h][e] = v > -FLT_MAX ? v : -FLT_MAX;
                }
        }

        if (POOL) {
            const int PW = W2, px0 = x0 >> 1, pc = tc >> 1; /* pooled columns of this tile */
            float *__restrict__ pstg = stg;
            if (a.out) CF_BARRIER(); /* the map's rows have been read */
            if (active) {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int p2 = wr * (8 * WC) + 8 * wx + 4 * h + g; /* pair of the tile's 64 pooled pixels */
                    *(float2 *)&pstg[(f * 32 + (p2 ^ (f << 1))) * 2] = make_float2(pooled[h][0], pooled[h][1]);
                }
                if (a.bits) {
                    /* one ballot per (h, e): its four 16-bit fields are the words of pooled columns 8h + 2g' + e */
                    unsigned word = 0;
#pragma unroll
                    for (int h = 0; h < 2; ++h)
#pragma unroll
                        for (int e = 0; e < 2; ++e) {
                            const unsigned long long m64 = __ballot(pooled[h][e] > 0.f);
#pragma unroll
                            for (int gg = 0; gg < 4; ++gg)
                                if (lane == 8 * h + 2 * gg + e) word = (unsigned)(m64 >> (16 * gg)) & 0xFFFFu;
                        }
                    if (M < 16) word &= (1u << M) - 1u;
                    if (lane < 16 && 16 * wx + lane < pc)
                        a.bits[((long)b * H2 + NRP * rp + wr) * PW + px0 + 16 * wx + lane] = word;
                }
            }
            CF_BARRIER();
            {
                const int m = tid >> 4, qq = tid & 15, pj = qq / (4 * WC), pq = qq % (4 * WC);
                if (4 * pq < pc && m < M) {
                    const float4 o = *(const float4 *)&pstg[(m * 16 + (qq ^ m)) * 4];
                    *(float4u *)(a.pool + (((long)b * M + m) * H2 + NRP * rp + pj) * PW + px0 + 4 * pq) =
                        (float4u){o.x, o.y, o.z, o.w};
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
        do_tile(patch0, patch1, stage);
        if (++t >= t_end) break;
        do_tile(patch1, patch0, stage);
        if (++t >= t_end) break;
    }
    __builtin_amdgcn_s_waitcnt(0); /* no wave ends with a direct-to-LDS load in flight */
}

/* Whether conv_first_kernel serves the layer (then also with the pooled outputs): 3x3 / stride 1 / pad 1
 * over 3 channels (up to 64 filters) or 16 channels (up to 32 filters: a lane keeps its filter's 144
 * weights in registers), even height, width a multiple of 8 (pooled rows leave in 16-byte quads). */
extern "C" int conv_first_serves(int batch, int c, int h, int w, int n, int groups, int size, int stride, int pad)
{
    if (groups != 1 || size != 3 || stride != 1 || pad != 1 || n < 1) return 0;
    if (!((c == 3 && n <= 64) || (c == 16 && n <= 32))) return 0;
    if (batch < 1 || h < 2 || (h & 1) || w < 32 || (w & 7)) return 0;
    if ((long)batch * c * h * w * 4 >= (1L << 32) - 64) return 0; /* 32-bit buffer offsets */
    if ((long)c * h * w * 4 >= (1L << 31)) return 0;              /* a lane's offsets inside one image are signed */
    if ((long)batch * (h / 2) * ((w + 31) / 32) >= (1L << 31)) return 0;
    return 1;
}

/* The tile shape, as waves side by side (4: 2 rows x 128 columns, 2: 4 x 64, 1: 8 x 32): among the
 * shapes whose height divides the image's, the one that wastes the fewest columns in the last tile of
 * a row (416 = 13 x 32 and 208 = 6.5 x 32 take the narrowest), the wider one on a tie.  With 16
 * channels the 2 x 128 tile's patch (4 rows x 136 columns x 16 channels, twice) leaves room for one
 * workgroup per CU only, so it is the last resort there.  The 2-row shape always applies.
 * g_shape != 0 forces a shape where the height allows it (tests, sweeps). */
static int g_shape = 0;

extern "C" void conv_first_set_shape(int waves_across) { g_shape = waves_across; }

static int shape_rows_fit(int wc, int h) { return h % (2 * (4 / wc)) == 0; }

static int pick_shape(int c, int h, int w)
{
    if ((g_shape == 4 || g_shape == 2 || g_shape == 1) && shape_rows_fit(g_shape, h)) return g_shape;
    int best = 4;
    double best_fill = -1.;
    for (int wc = 4; wc >= 1; wc >>= 1) {
        if (!shape_rows_fit(wc, h)) continue;
        const int cols = 32 * wc;
        double fill = (double)w / ((w + cols - 1) / cols * cols);
        if (c == 16 && wc == 4) fill *= 0.5;
        if (fill > best_fill + 1e-9) best_fill = fill, best = wc;
    }
    return best;
}

template <int TM, bool POOL, int C>
static const void *kernel_of_shape(int wc)
{
    return wc == 4 ? (const void *)conv_first_kernel<TM, POOL, 4, C>
         : wc == 2 ? (const void *)conv_first_kernel<TM, POOL, 2, C>
                   : (const void *)conv_first_kernel<TM, POOL, 1, C>;
}

template <bool POOL>
static const void *kernel16_of_shape(int wc)
{
    return wc == 4 ? (const void *)conv_first16_kernel<POOL, 4>
         : wc == 2 ? (const void *)conv_first16_kernel<POOL, 2>
                   : (const void *)conv_first16_kernel<POOL, 1>;
}

/* variant index: [3 channels, up to 16 filters | 16 channels | 3 channels, more than 32 filters | 3 channels, 17..32] */
static int variant_of(int c, int n) { return c == 16 ? 2 : n > 32 ? 1 : n <= 16 ? 3 : 0; }

/* Resident workgroups per CU of every variant [variant_of][pooled][shape], asked of the runtime once (from
 * the library's device set-up, so that no launch path has to: a caller may be capturing its stream). */
static int g_resident[4][2][3];

static const void *kernel_of(int v, int pooled, int wc)
{
    return v == 3 ? (pooled ? kernel16_of_shape<true>(wc) : kernel16_of_shape<false>(wc))
         : v == 2 ? (pooled ? kernel_of_shape<1, true, 16>(wc) : kernel_of_shape<1, false, 16>(wc))
         : v == 1 ? (pooled ? kernel_of_shape<2, true, 3>(wc) : kernel_of_shape<2, false, 3>(wc))
                  : (pooled ? kernel_of_shape<1, true, 3>(wc) : kernel_of_shape<1, false, 3>(wc));
}

extern "C" __attribute__((visibility("hidden"))) void conv_first_device_setup(void)
{
    if (g_resident[0][0][0]) return;
    for (int v = 3; v >= 0; --v) /* [0][0][0] last: it is the flag */
        for (int p = 1; p >= 0; --p)
            for (int s = 2; s >= 0; --s) {
                int nb = 0;
                hip_check_error(hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, kernel_of(v, p, 1 << s), CF_THREADS, 0));
                g_resident[v][p][s] = nb < 1 ? 1 : nb > 4 ? 4 : nb;
            }
}

extern "C" const char *conv_first_kernel_name(int c, int n, int pooled, int h, int w)
{
    static const char *const names[4][2][3] = {
        {{"conv_first_kernel<1,false,1,3>", "conv_first_kernel<1,false,2,3>", "conv_first_kernel<1,false,4,3>"},
         {"conv_first_kernel<1,true,1,3>", "conv_first_kernel<1,true,2,3>", "conv_first_kernel<1,true,4,3>"}},
        {{"conv_first_kernel<2,false,1,3>", "conv_first_kernel<2,false,2,3>", "conv_first_kernel<2,false,4,3>"},
         {"conv_first_kernel<2,true,1,3>", "conv_first_kernel<2,true,2,3>", "conv_first_kernel<2,true,4,3>"}},
        {{"conv_first_kernel<1,false,1,16>", "conv_first_kernel<1,false,2,16>", "conv_first_kernel<1,false,4,16>"},
         {"conv_first_kernel<1,true,1,16>", "conv_first_kernel<1,true,2,16>", "conv_first_kernel<1,true,4,16>"}},
        {{"conv_first16_kernel<false,1>", "conv_first16_kernel<false,2>", "conv_first16_kernel<false,4>"},
         {"conv_first16_kernel<true,1>", "conv_first16_kernel<true,2>", "conv_first16_kernel<true,4>"}}};
    const int wc = pick_shape(c, h, w);
    return names[variant_of(c, n)][pooled != 0][wc >> 1];
}

/* The launch.  `out` or `pool` may be null (not both); `bits` needs `pool`.  slope: the activation as
 * y > 0 ? y : slope*y.  start/stop: events to attach to the dispatch, or null. */
extern "C" void conv_first_forward(const float *input, const float *weights, const float *biases, const float *scales,
                                   const float *rolling_mean, const float *rolling_variance, float *out, float *pool,
                                   unsigned *bits, int batch, int c, int h, int w, int n, int batch_normalize,
                                   double slope, int cus, void *start, void *stop)
{
    if (!conv_first_serves(batch, c, h, w, n, 1, 3, 1, 1)) dn_fatal("conv_first_forward: geometry not served");
    if ((!out && !pool) || (bits && !pool)) dn_fatal("conv_first_forward: nothing to write");
    const int wc = pick_shape(c, h, w);
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
    a.in_bytes = (unsigned)((long)batch * c * h * w * 4);
    const dn_f2 s = dn_split(slope);
    a.slope_hi = s.hi;
    a.slope_lo = s.lo;
    const int v = variant_of(c, n);
    const void *kernel = kernel_of(v, pool != 0, wc);
    /* exactly as many workgroups as stay resident (two to four per CU, by the variant's registers and
     * LDS), each walking its run: one more per CU would start when the others end and run alone */
    if (!g_resident[0][0][0]) conv_first_device_setup();
    const int *per_cu = &g_resident[v][pool != 0][wc >> 1];
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
