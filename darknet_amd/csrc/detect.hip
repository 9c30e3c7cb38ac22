/*
 * detect.hip - the step right after the forward pass: thresholded decode of the yolo heads into
 * boxes and per-class non-maximum suppression, on the device, so that only the surviving
 * detections cross PCIe instead of the three full yolo tensors.
 *
 * A detection is a row of (5 + classes) floats: x, y, w, h, objectness, prob[classes].
 *
 * Decode follows get_yolo_detections (src/yolo_layer.c:316-343) with get_yolo_box (:83-91) and
 * correct_yolo_boxes (:247-273) folded in, including the reference's mixed float/double
 * arithmetic, and keeps the reference's order of detections (cells row-major, anchors inside a
 * cell): the threshold test is an ordered stream compaction, not an atomic append.
 * NMS follows do_nms_sort (src/box.c:58-89) with box_iou (:152-155): per class, detections in
 * descending probability suppress every later one that overlaps them by more than `thresh`.
 */
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "hip.h"

static inline hipStream_t dn_stream() { return (hipStream_t)hip_get_stream(); }

#define DN_DECODE_THREADS 1024
#define DN_MAX_ANCHORS 16

struct yolo_decode_args {
    const float *pred; /* one image's yolo output: [n][5 + classes][lh][lw] */
    float *rows;
    int *count;        /* running number of rows (device); this launch appends */
    int max_rows;
    int lw, lh, n, classes;
    int netw, neth, w, h, new_w, new_h, relative;
    float thresh;
    float anchors[2 * DN_MAX_ANCHORS]; /* biases[2*mask[i]], biases[2*mask[i]+1] */
};

/* Inclusive scan of one flag per thread over the workgroup; returns this thread's exclusive
 * prefix and the workgroup total. */
__device__ __forceinline__ int block_exclusive_scan(int flag, int *wave_sums, int &total)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned long long ballot = __ballot(flag);
    const int prefix = __popcll(ballot & ((1ull << lane) - 1ull));
    if (lane == 0) wave_sums[wave] = __popcll(ballot);
    __syncthreads();
    int base = 0, sum = 0;
    for (int i = 0; i < (int)(blockDim.x >> 6); ++i) {
        const int v = wave_sums[i];
        if (i < wave) base += v;
        sum += v;
    }
    __syncthreads();
    total = sum;
    return base + prefix;
}

__global__ __launch_bounds__(DN_DECODE_THREADS) void yolo_decode_kernel(yolo_decode_args a)
{
    __shared__ int wave_sums[DN_DECODE_THREADS / 64];
    const int cells = a.lw * a.lh;
    const int candidates = cells * a.n;
    const int entries = 5 + a.classes;
    int base = *a.count; /* written only by the last thread of this workgroup, at the end */
    for (int c0 = 0; c0 < candidates; c0 += DN_DECODE_THREADS) {
        const int c = c0 + (int)threadIdx.x;   /* candidate id = cell*n + anchor: the reference's loop order */
        const int cell = c / a.n, n = c - cell * a.n;
        float obj = 0.f;
        int keep = 0;
        if (c < candidates) {
            obj = a.pred[((long)n * entries + 4) * cells + cell];
            keep = obj > a.thresh;
        }
        int total;
        const int pos = base + block_exclusive_scan(keep, wave_sums, total);
        if (keep && pos < a.max_rows) {
            const float *p = a.pred + (long)n * entries * cells + cell;
            const int col = cell % a.lw, row = cell / a.lw;
            /* get_yolo_box: (i + x)/lw in float; exp() and the anchor product in double */
            float bx = __fdiv_rn(__fadd_rn((float)col, p[0]), (float)a.lw);
            float by = __fdiv_rn(__fadd_rn((float)row, p[(long)cells]), (float)a.lh);
            float bw = (float)(exp((double)p[2L * cells]) * (double)a.anchors[2 * n] / (double)a.netw);
            float bh = (float)(exp((double)p[3L * cells]) * (double)a.anchors[2 * n + 1] / (double)a.neth);
            /* correct_yolo_boxes */
            bx = (float)(((double)bx - (double)(a.netw - a.new_w) / 2. / (double)a.netw) /
                         (double)__fdiv_rn((float)a.new_w, (float)a.netw));
            by = (float)(((double)by - (double)(a.neth - a.new_h) / 2. / (double)a.neth) /
                         (double)__fdiv_rn((float)a.new_h, (float)a.neth));
            bw = __fmul_rn(bw, __fdiv_rn((float)a.netw, (float)a.new_w));
            bh = __fmul_rn(bh, __fdiv_rn((float)a.neth, (float)a.new_h));
            if (!a.relative) {
                bx = __fmul_rn(bx, (float)a.w);
                bw = __fmul_rn(bw, (float)a.w);
                by = __fmul_rn(by, (float)a.h);
                bh = __fmul_rn(bh, (float)a.h);
            }
            float *r = a.rows + (long)pos * entries;
            r[0] = bx;
            r[1] = by;
            r[2] = bw;
            r[3] = bh;
            r[4] = obj;
            for (int j = 0; j < a.classes; ++j) {
                const float prob = __fmul_rn(obj, p[(long)(5 + j) * cells]);
                r[5 + j] = (prob > a.thresh) ? prob : 0.f;
            }
        }
        base += total;
    }
    if (threadIdx.x == 0) *a.count = base; /* may exceed max_rows: the caller checks */
}

extern "C" void yolo_decode_gpu(const float *layer_output, int lw, int lh, int n, int classes,
                                const float *anchors, int netw, int neth, int w, int h, int relative,
                                float thresh, float *rows, int max_rows, int *count)
{
    if (!layer_output || !anchors || !rows || !count) dn_fatal("yolo_decode_gpu: null pointer");
    if (lw <= 0 || lh <= 0 || n <= 0 || classes < 0 || netw <= 0 || neth <= 0 || w <= 0 || h <= 0 || max_rows < 0)
        dn_fatal("yolo_decode_gpu: bad geometry");
    if (n > DN_MAX_ANCHORS) dn_fatal("yolo_decode_gpu: more than 16 anchors per head");
    yolo_decode_args a;
    a.pred = layer_output;
    a.rows = rows;
    a.count = count;
    a.max_rows = max_rows;
    a.lw = lw;
    a.lh = lh;
    a.n = n;
    a.classes = classes;
    a.netw = netw;
    a.neth = neth;
    a.w = w;
    a.h = h;
    a.relative = relative;
    a.thresh = thresh;
    /* the letterbox geometry of correct_yolo_boxes (src/yolo_layer.c:250-258), integer division */
    if (((float)netw / w) < ((float)neth / h)) {
        a.new_w = netw;
        a.new_h = (h * netw) / w;
    } else {
        a.new_h = neth;
        a.new_w = (w * neth) / h;
    }
    if (a.new_w <= 0 || a.new_h <= 0) dn_fatal("yolo_decode_gpu: image too thin for the network input");
    for (int i = 0; i < 2 * DN_MAX_ANCHORS; ++i) a.anchors[i] = i < 2 * n ? anchors[i] : 0.f;
    hipLaunchKernelGGL(yolo_decode_kernel, dim3(1), dim3(DN_DECODE_THREADS), 0, dn_stream(), a);
    dn_check_launch("yolo_decode_gpu");
}

/* ---- region head (yolov2): get_region_detections src/region_layer.c:364-437 ----------------
 * Every anchor of every cell becomes a row, at index anchor*cells + cell (no compaction: the
 * reference returns w*h*n detections); objectness below the threshold is stored as 0 and leaves
 * the class probabilities at 0.  Boxes: get_region_box :76-84 (anchors in cell units, divided
 * by the layer size) and correct_region_boxes :336-362. */
struct region_decode_args {
    const float *pred; /* one image's region output: [n][coords + 1 + classes][lh][lw] */
    float *rows;
    int *count;
    int max_rows;
    int lw, lh, n, classes, coords, background;
    int netw, neth, w, h, new_w, new_h, relative;
    float thresh;
    float anchors[2 * DN_MAX_ANCHORS];
};

__global__ void region_decode_kernel(region_decode_args a)
{
    const int cells = a.lw * a.lh;
    const int total = cells * a.n;
    const int entries = a.coords + a.classes + 1;
    const int base = *a.count;
    for (int idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += gridDim.x * blockDim.x) {
        if (base + idx >= a.max_rows) continue;
        const int n = idx / cells, cell = idx - n * cells;
        const int col = cell % a.lw, row = cell / a.lw;
        const float *p = a.pred + (long)n * entries * cells + cell;
        const float scale = a.background ? 1.f : p[(long)a.coords * cells];
        float bx = __fdiv_rn(__fadd_rn((float)col, p[0]), (float)a.lw);
        float by = __fdiv_rn(__fadd_rn((float)row, p[(long)cells]), (float)a.lh);
        float bw = (float)(exp((double)p[2L * cells]) * (double)a.anchors[2 * n] / (double)a.lw);
        float bh = (float)(exp((double)p[3L * cells]) * (double)a.anchors[2 * n + 1] / (double)a.lh);
        bx = (float)(((double)bx - (double)(a.netw - a.new_w) / 2. / (double)a.netw) /
                     (double)__fdiv_rn((float)a.new_w, (float)a.netw));
        by = (float)(((double)by - (double)(a.neth - a.new_h) / 2. / (double)a.neth) /
                     (double)__fdiv_rn((float)a.new_h, (float)a.neth));
        bw = __fmul_rn(bw, __fdiv_rn((float)a.netw, (float)a.new_w));
        bh = __fmul_rn(bh, __fdiv_rn((float)a.neth, (float)a.new_h));
        if (!a.relative) {
            bx = __fmul_rn(bx, (float)a.w);
            bw = __fmul_rn(bw, (float)a.w);
            by = __fmul_rn(by, (float)a.h);
            bh = __fmul_rn(bh, (float)a.h);
        }
        float *r = a.rows + (long)(base + idx) * (5 + a.classes);
        const float obj = scale > a.thresh ? scale : 0.f;
        r[0] = bx;
        r[1] = by;
        r[2] = bw;
        r[3] = bh;
        r[4] = obj;
        const float *cls = p + (long)(a.coords + 1) * cells;
        for (int j = 0; j < a.classes; ++j) {
            float v = 0.f;
            if (obj != 0.f) {
                const float prob = __fmul_rn(scale, cls[(long)j * cells]);
                v = (prob > a.thresh) ? prob : 0.f;
            }
            r[5 + j] = v;
        }
    }
}

__global__ void add_count_kernel(int *count, int n) { *count += n; }

extern "C" void region_decode_gpu(const float *layer_output, int lw, int lh, int n, int classes, int coords,
                                  int background, const float *anchors, int netw, int neth, int w, int h,
                                  int relative, float thresh, float *rows, int max_rows, int *count)
{
    if (!layer_output || !anchors || !rows || !count) dn_fatal("region_decode_gpu: null pointer");
    if (lw <= 0 || lh <= 0 || n <= 0 || classes < 0 || netw <= 0 || neth <= 0 || w <= 0 || h <= 0 || max_rows < 0)
        dn_fatal("region_decode_gpu: bad geometry");
    if (coords != 4) dn_fatal("region_decode_gpu: only coords=4 (no masks) is decoded");
    if (n > DN_MAX_ANCHORS) dn_fatal("region_decode_gpu: more than 16 anchors");
    region_decode_args a;
    a.pred = layer_output;
    a.rows = rows;
    a.count = count;
    a.max_rows = max_rows;
    a.lw = lw;
    a.lh = lh;
    a.n = n;
    a.classes = classes;
    a.coords = coords;
    a.background = background;
    a.netw = netw;
    a.neth = neth;
    a.w = w;
    a.h = h;
    a.relative = relative;
    a.thresh = thresh;
    if (((float)netw / w) < ((float)neth / h)) {
        a.new_w = netw;
        a.new_h = (h * netw) / w;
    } else {
        a.new_h = neth;
        a.new_w = (w * neth) / h;
    }
    if (a.new_w <= 0 || a.new_h <= 0) dn_fatal("region_decode_gpu: image too thin for the network input");
    for (int i = 0; i < 2 * DN_MAX_ANCHORS; ++i) a.anchors[i] = i < 2 * n ? anchors[i] : 0.f;
    const int total = lw * lh * n;
    hipLaunchKernelGGL(region_decode_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, dn_stream(), a);
    hipLaunchKernelGGL(add_count_kernel, dim3(1), dim3(1), 0, dn_stream(), count, total);
    dn_check_launch("region_decode_gpu");
}

/* ---- yolov1 detection layer --------------------------------------------------------------- */
struct detection_decode_args {
    const float *pred; /* one image: [cells][classes] probabilities, [cells][n] scales, [cells][n][4] boxes */
    float *rows;
    int *count;
    int max_rows;
    int side, n, classes, sqrt, w, h;
    float thresh;
};

/* get_detection_detections (src/detection_layer.c:225-252) in its own arithmetic: the centre in
 * float, the extent through pow() in double (pow(x, 2) of a float is the exact product, pow(x, 1)
 * is x).  The objectness is stored whatever the threshold, as there. */
__global__ void detection_decode_kernel(detection_decode_args a)
{
    const int cells = a.side * a.side;
    const int total = cells * a.n;
    const int base = *a.count;
    for (int idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += gridDim.x * blockDim.x) {
        if (base + idx >= a.max_rows) continue;
        const int cell = idx / a.n;
        const int row = cell / a.side, col = cell - row * a.side;
        const float scale = a.pred[cells * a.classes + idx];
        const float *bx = a.pred + cells * (a.classes + a.n) + idx * 4;
        const double wd = (double)bx[2], hd = (double)bx[3];
        float *r = a.rows + (long)(base + idx) * (5 + a.classes);
        r[0] = __fmul_rn(__fdiv_rn(__fadd_rn(bx[0], (float)col), (float)a.side), (float)a.w);
        r[1] = __fmul_rn(__fdiv_rn(__fadd_rn(bx[1], (float)row), (float)a.side), (float)a.h);
        r[2] = (float)((a.sqrt ? wd * wd : wd) * (double)a.w);
        r[3] = (float)((a.sqrt ? hd * hd : hd) * (double)a.h);
        r[4] = scale;
        const float *cls = a.pred + cell * a.classes;
        for (int j = 0; j < a.classes; ++j) {
            const float prob = __fmul_rn(scale, cls[j]);
            r[5 + j] = (prob > a.thresh) ? prob : 0.f;
        }
    }
}

extern "C" void detection_decode_gpu(const float *layer_output, int side, int n, int classes, int sqrt, int w,
                                     int h, float thresh, float *rows, int max_rows, int *count)
{
    if (!layer_output || !rows || !count) dn_fatal("detection_decode_gpu: null pointer");
    if (side <= 0 || n <= 0 || classes < 0 || w <= 0 || h <= 0 || max_rows < 0 ||
        (long)side * side * ((long)n * 5 + classes) > 0x7fffffffL)
        dn_fatal("detection_decode_gpu: bad geometry");
    detection_decode_args a;
    a.pred = layer_output;
    a.rows = rows;
    a.count = count;
    a.max_rows = max_rows;
    a.side = side;
    a.n = n;
    a.classes = classes;
    a.sqrt = sqrt;
    a.w = w;
    a.h = h;
    a.thresh = thresh;
    const int total = side * side * n;
    hipLaunchKernelGGL(detection_decode_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, dn_stream(), a);
    hipLaunchKernelGGL(add_count_kernel, dim3(1), dim3(1), 0, dn_stream(), count, total);
    dn_check_launch("detection_decode_gpu");
}

/* ---- non-maximum suppression ------------------------------------------------------------- */
/* box_iou of src/box.c:111-155 in the reference's float arithmetic */
__device__ __forceinline__ float dn_overlap(float x1, float w1, float x2, float w2)
{
    const float l1 = __fsub_rn(x1, __fdiv_rn(w1, 2.f)), l2 = __fsub_rn(x2, __fdiv_rn(w2, 2.f));
    const float left = l1 > l2 ? l1 : l2;
    const float r1 = __fadd_rn(x1, __fdiv_rn(w1, 2.f)), r2 = __fadd_rn(x2, __fdiv_rn(w2, 2.f));
    const float right = r1 < r2 ? r1 : r2;
    return __fsub_rn(right, left);
}

__device__ __forceinline__ float dn_box_iou(const float *a, const float *b)
{
    const float w = dn_overlap(a[0], a[2], b[0], b[2]);
    const float h = dn_overlap(a[1], a[3], b[1], b[3]);
    const float inter = (w < 0 || h < 0) ? 0.f : __fmul_rn(w, h);
    const float uni = __fsub_rn(__fadd_rn(__fmul_rn(a[2], a[3]), __fmul_rn(b[2], b[3])), inter);
    return __fdiv_rn(inter, uni);
}

#define DN_NMS_THREADS 256

/* One workgroup per class.  Only detections with a nonzero probability for the class take part
 * (a zero one neither suppresses nor can be suppressed any further), so the work per class is
 * the handful of candidates of that class:
 *   1. ordered compaction of their indices,
 *   2. rank sort by descending probability (ties: lower index first; the reference's qsort
 *      leaves the order of ties unspecified),
 *   3. the greedy sweep: the next live candidate clears every later one it overlaps. */
__global__ __launch_bounds__(DN_NMS_THREADS) void nms_class_kernel(float *rows, int total, int classes,
                                                                    float thresh, int *idx, int *sorted,
                                                                    int *alive)
{
    __shared__ int wave_sums[DN_NMS_THREADS / 64];
    __shared__ int s_live;
    const int k = blockIdx.x;
    const int entries = 5 + classes;
    idx += (long)k * total;
    sorted += (long)k * total;
    alive += (long)k * total;
    int n = 0;
    for (int i0 = 0; i0 < total; i0 += DN_NMS_THREADS) {
        const int i = i0 + (int)threadIdx.x;
        const int keep = i < total && rows[(long)i * entries + 5 + k] != 0.f;
        int tot;
        const int pos = n + block_exclusive_scan(keep, wave_sums, tot);
        if (keep) idx[pos] = i;
        n += tot;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < n; e += DN_NMS_THREADS) {
        const float pe = rows[(long)idx[e] * entries + 5 + k];
        int rank = 0;
        for (int f = 0; f < n; ++f) {
            const float pf = rows[(long)idx[f] * entries + 5 + k];
            rank += (pf > pe) || (pf == pe && f < e);
        }
        sorted[rank] = idx[e];
        alive[rank] = 1;
    }
    __syncthreads();
    for (int s = 0; s < n; ++s) {
        if (threadIdx.x == 0) s_live = alive[s];
        __syncthreads();
        const int live = s_live;
        if (live) {
            const float *a = rows + (long)sorted[s] * entries;
            for (int t = s + 1 + (int)threadIdx.x; t < n; t += DN_NMS_THREADS)
                if (alive[t] && dn_box_iou(a, rows + (long)sorted[t] * entries) > thresh) alive[t] = 0;
        }
        __syncthreads();
    }
    for (int t = threadIdx.x; t < n; t += DN_NMS_THREADS)
        if (!alive[t]) rows[(long)sorted[t] * entries + 5 + k] = 0.f;
}

static int *g_nms_scratch = 0;
static size_t g_nms_scratch_ints = 0;

extern "C" void nms_sort_gpu(float *rows, int total, int classes, float thresh)
{
    if (total <= 0 || classes <= 0) return;
    if (!rows) dn_fatal("nms_sort_gpu: null pointer");
    const size_t need = (size_t)3 * classes * total;
    if (need > g_nms_scratch_ints) {
        if (g_nms_scratch) hip_free((float *)g_nms_scratch);
        g_nms_scratch = hip_make_int_array(0, need);
        g_nms_scratch_ints = need;
    }
    int *idx = g_nms_scratch, *sorted = idx + (size_t)classes * total, *alive = sorted + (size_t)classes * total;
    hipLaunchKernelGGL(nms_class_kernel, dim3((unsigned)classes), dim3(DN_NMS_THREADS), 0, dn_stream(), rows,
                       total, classes, thresh, idx, sorted, alive);
    dn_check_launch("nms_sort_gpu");
}
