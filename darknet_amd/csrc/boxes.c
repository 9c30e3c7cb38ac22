/*
 * boxes.c - detections out of a forwarded network: the reference's get_network_boxes /
 * do_nms_sort / free_detections (src/network.c:510-583, src/box.c:58-89) with the arithmetic
 * on the device (detect.hip).  The yolo heads are decoded where they lie in device memory; only
 * the thresholded rows come back to the host.
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "host.h"

/* Worst case number of rows: every anchor of every cell of every yolo head. */
static int network_max_detections(network *net, int *classes)
{
    int i, s = 0, cl = -1;
    for (i = 0; i < net->n; ++i) {
        layer l = net->layers[i];
        if (l.type != YOLO && l.type != REGION && l.type != DETECTION) continue;
        s += l.w * l.h * l.n;
        if (cl >= 0 && cl != l.classes) dn_fatal("detections: heads disagree on the number of classes");
        cl = l.classes;
    }
    if (classes) *classes = cl < 0 ? 0 : cl;
    return s;
}

static void ensure_detection_buffers(network *net)
{
    int classes, rows = network_max_detections(net, &classes);
    if (net->det_rows_gpu && net->det_max_rows >= rows) return;
    if (net->det_rows_gpu) hip_free(net->det_rows_gpu);
    if (net->det_count_gpu) hip_free((float *)net->det_count_gpu);
    net->det_rows_gpu = hip_make_array(0, (size_t)(rows > 0 ? rows : 1) * (size_t)(5 + classes));
    net->det_count_gpu = hip_make_int_array(0, 1);
    net->det_max_rows = rows;
}

/* Decodes every yolo head of image `b` into net->det_rows_gpu, in layer order as
 * fill_network_boxes (src/network.c:543-561) concatenates them.  Returns the number of rows. */
int network_decode_image_gpu(network *net, int b, int w, int h, float thresh, int relative)
{
    int i, j, count = 0;
    if (b < 0 || b >= net->batch) dn_fatal("detections: image index outside the batch");
    ensure_detection_buffers(net);
    hip_push_int_array(net->det_count_gpu, &count, 1);
    for (i = 0; i < net->n; ++i) {
        layer l = net->layers[i];
        float anchors[32];
        if (l.type == DETECTION) { /* src/network.c:555-558 */
            detection_decode_gpu(l.output_gpu + (size_t)b * l.outputs, l.side, l.n, l.classes, l.sqrt, w, h, thresh,
                                 net->det_rows_gpu, net->det_max_rows, net->det_count_gpu);
            continue;
        }
        if (l.type != YOLO && l.type != REGION) continue;
        if (l.n > 16) dn_fatal("detections: more than 16 anchors per head");
        if (l.type == REGION) { /* src/network.c:553-556 */
            region_decode_gpu(l.output_gpu + (size_t)b * l.outputs, l.w, l.h, l.n, l.classes, l.coords,
                              l.background, l.biases, net->w, net->h, w, h, relative, thresh, net->det_rows_gpu,
                              net->det_max_rows, net->det_count_gpu);
            continue;
        }
        for (j = 0; j < l.n; ++j) {
            anchors[2 * j] = l.biases[2 * l.mask[j]];
            anchors[2 * j + 1] = l.biases[2 * l.mask[j] + 1];
        }
        yolo_decode_gpu(l.output_gpu + (size_t)b * l.outputs, l.w, l.h, l.n, l.classes, anchors, net->w, net->h,
                        w, h, relative, thresh, net->det_rows_gpu, net->det_max_rows, net->det_count_gpu);
    }
    hip_pull_int_array(net->det_count_gpu, &count, 1);
    if (count > net->det_max_rows) dn_fatal("detections: row buffer overflow");
    return count;
}

/* src/network.c:510-524: how many boxes get_network_boxes would return (image 0) */
int num_detections(network *net, float thresh)
{
    return network_decode_image_gpu(net, 0, net->w, net->h, thresh, 1);
}

static detection *alloc_detections(int n, int classes)
{
    int i;
    detection *dets = (detection *)dn_calloc((size_t)(n > 0 ? n : 1), sizeof(detection));
    for (i = 0; i < n; ++i) dets[i].prob = (float *)dn_calloc((size_t)(classes > 0 ? classes : 1), sizeof(float));
    return dets;
}

/* src/network.c:526-541 */
detection *make_network_boxes(network *net, float thresh, int *num)
{
    int classes, n = num_detections(net, thresh);
    network_max_detections(net, &classes);
    if (num) *num = n;
    return alloc_detections(n, classes);
}

static void rows_to_detections(const float *rows, int n, int classes, detection *dets)
{
    int i;
    for (i = 0; i < n; ++i) {
        const float *r = rows + (size_t)i * (5 + classes);
        dets[i].bbox.x = r[0];
        dets[i].bbox.y = r[1];
        dets[i].bbox.w = r[2];
        dets[i].bbox.h = r[3];
        dets[i].objectness = r[4];
        dets[i].classes = classes;
        memcpy(dets[i].prob, r + 5, sizeof(float) * (size_t)classes);
    }
}

static void pull_rows(network *net, int n, int classes, detection *dets)
{
    float *rows;
    if (n <= 0) return;
    rows = (float *)dn_calloc((size_t)n * (5 + classes), sizeof(float));
    hip_pull_array(net->det_rows_gpu, rows, (size_t)n * (5 + classes));
    rows_to_detections(rows, n, classes, dets);
    free(rows);
}

/* src/network.c:543-561; `dets` must come from make_network_boxes with the same threshold */
void fill_network_boxes(network *net, int w, int h, float thresh, float hier, int *map, int relative,
                        detection *dets)
{
    int classes, n;
    (void)hier;
    if (map) dn_fatal("fill_network_boxes: map is not supported");
    network_max_detections(net, &classes);
    n = network_decode_image_gpu(net, 0, w, h, thresh, relative);
    pull_rows(net, n, classes, dets);
}

/* get_network_boxes for image `b` of the batch (the reference only ever looks at image 0,
 * src/yolo_layer.c:326), optionally followed by do_nms_sort on the device (nms > 0) so that the
 * rows cross PCIe once, after suppression. */
detection *get_network_boxes_image(network *net, int b, int w, int h, float thresh, int relative, float nms,
                                   int *num)
{
    int classes, n;
    detection *dets;
    network_max_detections(net, &classes);
    n = network_decode_image_gpu(net, b, w, h, thresh, relative);
    if (nms > 0 && n > 0) nms_sort_gpu(net->det_rows_gpu, n, classes, nms);
    dets = alloc_detections(n, classes);
    pull_rows(net, n, classes, dets);
    if (num) *num = n;
    return dets;
}

/* src/network.c:563-568 */
detection *get_network_boxes(network *net, int w, int h, float thresh, float hier, int *map, int relative,
                             int *num)
{
    (void)hier;
    if (map) dn_fatal("get_network_boxes: map is not supported");
    return get_network_boxes_image(net, 0, w, h, thresh, relative, 0.f, num);
}

/* src/network.c:570-579 */
void free_detections(detection *dets, int n)
{
    int i;
    if (!dets) return;
    for (i = 0; i < n; ++i) {
        free(dets[i].prob);
        if (dets[i].mask) free(dets[i].mask);
    }
    free(dets);
}

/* src/box.c:58-89.  Per class, in descending probability, a detection zeroes the class
 * probability of every later one whose box overlaps it by more than `thresh`.  The array keeps
 * its order (the reference leaves it sorted by the last class, ties in unspecified order);
 * detections with objectness 0 are moved to the end as the reference does. */
void do_nms_sort(detection *dets, int total, int classes, float thresh)
{
    int i, k;
    float *rows, *rows_gpu;
    k = total - 1;
    for (i = 0; i <= k; ++i) {
        if (dets[i].objectness == 0) {
            detection swap = dets[i];
            dets[i] = dets[k];
            dets[k] = swap;
            --k;
            --i;
        }
    }
    total = k + 1;
    if (total <= 0 || classes <= 0) return;
    rows = (float *)dn_calloc((size_t)total * (5 + classes), sizeof(float));
    for (i = 0; i < total; ++i) {
        float *r = rows + (size_t)i * (5 + classes);
        r[0] = dets[i].bbox.x;
        r[1] = dets[i].bbox.y;
        r[2] = dets[i].bbox.w;
        r[3] = dets[i].bbox.h;
        r[4] = dets[i].objectness;
        memcpy(r + 5, dets[i].prob, sizeof(float) * (size_t)classes);
    }
    rows_gpu = hip_make_array(rows, (size_t)total * (5 + classes));
    nms_sort_gpu(rows_gpu, total, classes, thresh);
    hip_pull_array(rows_gpu, rows, (size_t)total * (5 + classes));
    hip_free(rows_gpu);
    for (i = 0; i < total; ++i)
        memcpy(dets[i].prob, rows + (size_t)i * (5 + classes) + 5, sizeof(float) * (size_t)classes);
    free(rows);
}
