/*
 * images.c - the reference's image calls on the input side of the path (make_image, free_image,
 * resize_image, letterbox_image: src/image.c; network_predict_image: src/network.c:579-586)
 * with the arithmetic on the device (image.hip), plus the form the device wants: a frame goes
 * up once at its own size, through a pinned staging buffer and an asynchronous copy on the
 * launch stream, and is letterboxed straight into its slot of the network's input buffer.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <hip/hip_runtime_api.h>

#include "host.h"

/* src/image.c:734-748 */
image make_empty_image(int w, int h, int c)
{
    image out;
    out.data = 0;
    out.h = h;
    out.w = w;
    out.c = c;
    return out;
}

image make_image(int w, int h, int c)
{
    image out = make_empty_image(w, h, c);
    out.data = (float *)dn_calloc((size_t)h * w * c, sizeof(float));
    return out;
}

/* src/image.c:1368-1373 */
void free_image(image m)
{
    if (m.data) free(m.data);
}

/* Pinned staging and device scratch, grown on demand and kept for the life of the process. */
static float *g_stage = 0, *g_frame_gpu = 0;
static size_t g_stage_floats = 0, g_frame_floats = 0;

static float *upload_frame(image im)
{
    const size_t n = (size_t)im.w * im.h * im.c;
    if (!im.data || im.w <= 0 || im.h <= 0 || im.c <= 0) dn_fatal("image: empty image");
    /* the staging buffer may still feed the previous frame's copy */
    hip_synchronize();
    if (n > g_stage_floats) {
        if (g_stage) hip_check_error((int)hipHostFree(g_stage));
        hip_check_error((int)hipHostMalloc((void **)&g_stage, n * sizeof(float), hipHostMallocDefault));
        g_stage_floats = n;
    }
    if (n > g_frame_floats) {
        if (g_frame_gpu) hip_free(g_frame_gpu);
        g_frame_gpu = hip_make_array(0, n);
        g_frame_floats = n;
    }
    memcpy(g_stage, im.data, n * sizeof(float));
    hip_check_error((int)hipMemcpyAsync(g_frame_gpu, g_stage, n * sizeof(float), hipMemcpyHostToDevice,
                                        (hipStream_t)hip_get_stream()));
    return g_frame_gpu;
}

/* src/image.c:1199-1241: host image in, host image out, computed on the device */
image resize_image(image im, int w, int h)
{
    image out = make_image(w, h, im.c);
    float *src = upload_frame(im);
    float *dst = hip_make_array(0, (size_t)w * h * im.c);
    resize_image_gpu(src, im.w, im.h, im.c, dst, w, h);
    hip_pull_array(dst, out.data, (size_t)w * h * im.c);
    hip_free(dst);
    return out;
}

/* src/image.c:812-831 */
image letterbox_image(image im, int w, int h)
{
    image out = make_image(w, h, im.c);
    float *src = upload_frame(im);
    float *dst = hip_make_array(0, (size_t)w * h * im.c);
    letterbox_image_gpu(src, im.w, im.h, im.c, dst, w, h);
    hip_pull_array(dst, out.data, (size_t)w * h * im.c);
    hip_free(dst);
    return out;
}

/* Letterboxes `im` into image slot b of the network's device input (no host round trip). */
void network_letterbox_input(network *net, int b, image im)
{
    if (b < 0 || b >= net->batch) dn_fatal("network_letterbox_input: image index outside the batch");
    if (im.c != net->c) dn_fatal("network_letterbox_input: channel count differs from the network's");
    if (!(net->w && net->h && net->c)) dn_fatal("network_letterbox_input: the network input is not an image");
    letterbox_image_gpu(upload_frame(im), im.w, im.h, im.c, net->input_gpu + (size_t)b * net->inputs, net->w,
                        net->h);
}

/* src/network.c:579-586: letterbox, batch 1, forward; the result is the host copy of the
 * output layer as after network_predict */
float *network_predict_image(network *net, image im)
{
    set_batch_network(net, 1);
    network_letterbox_input(net, 0, im);
    forward_network_device(net);
    network_pull_outputs(net);
    return net->output;
}
