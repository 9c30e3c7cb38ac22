/*
 * image.hip - the input side of the path: bilinear resize and letterbox of an image, on the
 * device, so that a frame is uploaded once at its own size and lands in the network's input
 * buffer without a host-side resize or a second copy.
 *
 * resize_image (src/image.c:1199-1241) is a separable bilinear filter done in two passes with a
 * float intermediate: a horizontal pass into `part`, then a vertical pass.  Both passes are
 * reproduced operation by operation (products rounded, then added), with the horizontal values
 * recomputed where the vertical pass needs them instead of being stored, so the result equals
 * the reference's bit for bit.  letterbox_image (:812-831) fills the target with .5 and embeds
 * the resized image centred (embed_image :428-439).
 */
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "hip.h"

static inline hipStream_t dn_stream() { return (hipStream_t)hip_get_stream(); }

#define DN_BLOCK 256

struct resize_args {
    const float *im;
    float *out;
    int w, h, c;          /* source */
    int rw, rh;           /* resized */
    int ow, oh;           /* destination plane (== rw, rh for a plain resize) */
    int dx, dy;           /* where the resized image sits in the destination */
    float w_scale, h_scale;
    float fill;
    int letterbox;
};

/* one value of the horizontal pass: `part` at column cx of source row y, channel plane p */
__device__ __forceinline__ float resize_row(const resize_args &a, const float *plane, int cx, int y)
{
    const float *row = plane + (long)y * a.w;
    if (cx == a.rw - 1 || a.w == 1) return row[a.w - 1];
    const float sx = __fmul_rn((float)cx, a.w_scale);
    const int ix = (int)sx;
    const float dx = __fsub_rn(sx, (float)ix);
    return __fadd_rn(__fmul_rn(__fsub_rn(1.f, dx), row[ix]), __fmul_rn(dx, row[ix + 1]));
}

__global__ void resize_kernel(resize_args a)
{
    const long n = (long)a.ow * a.oh * a.c;
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        const int x = (int)(i % a.ow);
        long t = i / a.ow;
        const int y = (int)(t % a.oh);
        const int k = (int)(t / a.oh);
        const int cx = x - a.dx, ry = y - a.dy;
        if (cx < 0 || cx >= a.rw || ry < 0 || ry >= a.rh) {
            if (a.letterbox) a.out[i] = a.fill;
            continue;
        }
        const float *plane = a.im + (long)k * a.h * a.w;
        const float sy = __fmul_rn((float)ry, a.h_scale);
        const int iy = (int)sy;
        const float dy = __fsub_rn(sy, (float)iy);
        float val = __fmul_rn(__fsub_rn(1.f, dy), resize_row(a, plane, cx, iy));
        if (!(ry == a.rh - 1 || a.h == 1)) val = __fadd_rn(val, __fmul_rn(dy, resize_row(a, plane, cx, iy + 1)));
        a.out[i] = val;
    }
}

static void launch_resize(const float *im, int w, int h, int c, float *out, int rw, int rh, int ow, int oh, int dx,
                          int dy, int letterbox, const char *what)
{
    if (!im || !out) dn_fatal("resize: null pointer");
    if (w <= 0 || h <= 0 || c <= 0 || rw <= 0 || rh <= 0) dn_fatal("resize: bad geometry");
    /* the reference divides by (w-1) and (h-1): a one-pixel-wide or -high result is only
     * defined when the source has that extent too */
    if ((rw == 1 && w != 1) || (rh == 1 && h != 1)) dn_fatal("resize: a 1-pixel extent needs a 1-pixel source");
    resize_args a;
    a.im = im;
    a.out = out;
    a.w = w;
    a.h = h;
    a.c = c;
    a.rw = rw;
    a.rh = rh;
    a.ow = ow;
    a.oh = oh;
    a.dx = dx;
    a.dy = dy;
    a.w_scale = rw > 1 ? (float)(w - 1) / (rw - 1) : 0.f;
    a.h_scale = rh > 1 ? (float)(h - 1) / (rh - 1) : 0.f;
    a.fill = .5f;
    a.letterbox = letterbox;
    const long n = (long)ow * oh * c;
    long blocks = (n + DN_BLOCK - 1) / DN_BLOCK;
    if (blocks > 256L * 32) blocks = 256L * 32;
    hipLaunchKernelGGL(resize_kernel, dim3((unsigned)blocks), dim3(DN_BLOCK), 0, dn_stream(), a);
    dn_check_launch(what);
}

extern "C" void resize_image_gpu(const float *im, int w, int h, int c, float *out, int out_w, int out_h)
{
    launch_resize(im, w, h, c, out, out_w, out_h, out_w, out_h, 0, 0, 0, "resize_image_gpu");
}

extern "C" void letterbox_image_gpu(const float *im, int w, int h, int c, float *boxed, int box_w, int box_h)
{
    int new_w, new_h;
    if (box_w <= 0 || box_h <= 0 || w <= 0 || h <= 0) dn_fatal("letterbox_image_gpu: bad geometry");
    if (((float)box_w / w) < ((float)box_h / h)) { /* src/image.c:816-822, integer division */
        new_w = box_w;
        new_h = (h * box_w) / w;
    } else {
        new_h = box_h;
        new_w = (w * box_h) / h;
    }
    if (new_w < 1 || new_h < 1) dn_fatal("letterbox_image_gpu: image too thin for the box");
    launch_resize(im, w, h, c, boxed, new_w, new_h, box_w, box_h, (box_w - new_w) / 2, (box_h - new_h) / 2, 1,
                  "letterbox_image_gpu");
}
