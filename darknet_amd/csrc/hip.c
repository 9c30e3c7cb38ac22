/*
 * hip.c - device shim of the darknet forward path on HIP.  Takes the place of the reference's
 * src/cuda.c: device selection, allocation, host<->device copies, error check.  There is no
 * BLAS/DNN handle here on purpose: the convolution is this library's own kernel.
 */
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "hip.h"

int gpu_index = 0;

static hipStream_t g_stream = 0;
static char g_name[640];

void dn_fatal(const char *msg)
{
    fprintf(stderr, "darknet-hip: %s\n", msg);
    fflush(stderr);
    exit(-1);
}

void hip_check_error(int status)
{
    if (status != hipSuccess) {
        char buf[320];
        snprintf(buf, sizeof buf, "HIP Error: %s", hipGetErrorString((hipError_t)status));
        dn_fatal(buf);
    }
    hipError_t prev = hipGetLastError();
    if (prev != hipSuccess) {
        char buf[320];
        snprintf(buf, sizeof buf, "HIP Error Prev: %s", hipGetErrorString(prev));
        dn_fatal(buf);
    }
}

void dn_check_launch(const char *what)
{
    hipError_t e = hipPeekAtLastError();
    if (e != hipSuccess) {
        char buf[384];
        snprintf(buf, sizeof buf, "kernel launch failed (%s): %s", what, hipGetErrorString(e));
        dn_fatal(buf);
    }
}

/* Parse-only mode: cfg parsing, layer tables and weights-file reading/writing work on host memory
 * alone (a machine without a GPU can inspect a network); nothing is allocated on or copied to a
 * device, and every entry point that would launch work ends the process instead of computing
 * anything on the host. */
static int g_parse_only = 0;
void hip_set_parse_only(int on) { g_parse_only = on ? 1 : 0; }
int hip_parse_only(void) { return g_parse_only; }
void hip_require_device(const char *what)
{
    if (g_parse_only) {
        fprintf(stderr, "%s: the library is in parse-only mode, no device work is possible\n", what);
        exit(-1);
    }
}

/* conv_mfma.hip: per-device set-up of the convolution dispatcher (CU count, address of the fixed
 * scratch array of the allocation-free entry point) */
void conv_device_setup(void);

void hip_set_device(int n)
{
    gpu_index = n;
    if (g_parse_only) return;
    hip_check_error(hipSetDevice(n));
    conv_device_setup();
}

int hip_get_device(void)
{
    int n = 0;
    hip_check_error(hipGetDevice(&n));
    return n;
}

const char *hip_device_name(void)
{
    hipDeviceProp_t p;
    hip_check_error(hipGetDeviceProperties(&p, hip_get_device()));
    snprintf(g_name, sizeof g_name, "%s (%s, %d CUs)", p.name, p.gcnArchName, p.multiProcessorCount);
    return g_name;
}

void *hip_get_stream(void) { return (void *)g_stream; }
void hip_set_stream(void *stream) { g_stream = (hipStream_t)stream; }

void hip_synchronize(void)
{
    hip_check_error(hipStreamSynchronize(g_stream));
}

float *hip_make_array(float *x, size_t n)
{
    float *x_gpu = 0;
    size_t size = sizeof(float) * (n ? n : 1);
    if (g_parse_only) return 0;
    hip_check_error(hipMalloc((void **)&x_gpu, size));
    if (!x_gpu) dn_fatal("hipMalloc returned a null pointer");
    if (x) {
        hip_check_error(hipMemcpy(x_gpu, x, sizeof(float) * n, hipMemcpyHostToDevice));
    } else {
        hip_check_error(hipMemset(x_gpu, 0, size));
    }
    return x_gpu;
}

int *hip_make_int_array(int *x, size_t n)
{
    int *x_gpu = 0;
    size_t size = sizeof(int) * (n ? n : 1);
    if (g_parse_only) return 0;
    hip_check_error(hipMalloc((void **)&x_gpu, size));
    if (!x_gpu) dn_fatal("hipMalloc returned a null pointer");
    if (x) hip_check_error(hipMemcpy(x_gpu, x, sizeof(int) * n, hipMemcpyHostToDevice));
    else hip_check_error(hipMemset(x_gpu, 0, size));
    return x_gpu;
}

/* Packed-weights cache for binders whose `layer` has no member for the packed copy (a darknet tree
 * that keeps the reference's struct): keyed by the device address of the weights and the layer's
 * geometry.  An entry is dropped when its weights are freed through hip_free or written through
 * hip_push_array, so a cached copy is never older than the weights it was made from as long as
 * the weights change through this shim (inference does not change them any other way).  Like the
 * reference's per-device handles (src/cuda.c:67-68,80-81) the table is not synchronised: one host
 * thread at a time. */
typedef struct {
    const float *weights;
    float *packed;
    size_t nweights;
    int n, c, groups, size;
} packed_entry;
static packed_entry *g_packed = 0;
static int g_npacked = 0, g_cap_packed = 0;

static void packed_drop_range(const float *lo, size_t n)
{
    int i = 0;
    while (i < g_npacked) {
        const float *w = g_packed[i].weights;
        if (w + g_packed[i].nweights > lo && w < lo + (n ? n : 1)) {
            hip_check_error(hipFree(g_packed[i].packed));
            g_packed[i] = g_packed[--g_npacked];
        } else {
            ++i;
        }
    }
}

void conv_packed_forget(const float *weights)
{
    if (g_npacked) packed_drop_range(weights, 1);
}

int conv_packed_cached_count(void) { return g_npacked; }

const float *conv_packed_cached_gpu(const float *weights, int n, int c, int groups, int size)
{
    const size_t floats = conv_packed_floats(n, c, groups, size);
    packed_entry e;
    int i;
    if (!floats) return 0;
    hip_require_device("conv_packed_cached_gpu");
    for (i = 0; i < g_npacked; ++i) {
        const packed_entry *p = &g_packed[i];
        if (p->weights == weights) {
            if (p->n == n && p->c == c && p->groups == groups && p->size == size) return p->packed;
            break; /* same address, another layer: the old copy belongs to freed weights */
        }
    }
    conv_packed_forget(weights);
    e.weights = weights;
    e.nweights = (size_t)n * (size_t)(c / groups) * (size_t)size * (size_t)size;
    e.n = n;
    e.c = c;
    e.groups = groups;
    e.size = size;
    e.packed = hip_make_array(0, floats);
    conv_pack_weights_gpu(weights, e.packed, n, c, groups, size);
    if (g_npacked == g_cap_packed) {
        g_cap_packed = g_cap_packed ? 2 * g_cap_packed : 64;
        g_packed = realloc(g_packed, sizeof(*g_packed) * (size_t)g_cap_packed);
        if (!g_packed) dn_fatal("Malloc error");
    }
    g_packed[g_npacked++] = e;
    return e.packed;
}

void hip_free(float *x_gpu)
{
    if (g_parse_only) return;
    if (g_npacked && x_gpu) packed_drop_range(x_gpu, 1);
    hip_check_error(hipFree(x_gpu));
}

/* Pinned host buffers for what network_predict hands back (yolo / region / last-layer outputs):
 * a copy into pinned memory is one DMA at the link's rate, where pageable memory has to pass
 * through the staging buffers below at the speed of a host memcpy.  The library remembers its own
 * pinned blocks so that push/pull recognise them; anything else is treated as pageable. */
static struct { char *p; size_t bytes; } *g_pinned = 0;
static int g_npinned = 0, g_cap_pinned = 0;

float *hip_host_alloc(size_t n)
{
    const size_t bytes = sizeof(float) * (n ? n : 1);
    void *p = 0;
    if (g_parse_only || hipHostMalloc(&p, bytes, hipHostMallocDefault) != hipSuccess || !p) {
        (void)hipGetLastError(); /* the failed allocation must not surface at the next launch check */
        p = calloc(1, bytes);
        if (!p) dn_fatal("Malloc error");
        return (float *)p;
    }
    memset(p, 0, bytes);
    if (g_npinned == g_cap_pinned) {
        g_cap_pinned = g_cap_pinned ? 2 * g_cap_pinned : 16;
        g_pinned = realloc(g_pinned, sizeof(*g_pinned) * (size_t)g_cap_pinned);
        if (!g_pinned) dn_fatal("Malloc error");
    }
    g_pinned[g_npinned].p = (char *)p;
    g_pinned[g_npinned].bytes = bytes;
    ++g_npinned;
    return (float *)p;
}

void hip_host_free(float *x)
{
    int i;
    if (!x) return;
    for (i = 0; i < g_npinned; ++i)
        if (g_pinned[i].p == (char *)x) {
            hip_check_error(hipHostFree(x));
            g_pinned[i] = g_pinned[--g_npinned];
            return;
        }
    free(x);
}

int dn_host_is_pinned(const void *x, size_t bytes)
{
    int i;
    for (i = 0; i < g_npinned; ++i)
        if ((const char *)x >= g_pinned[i].p && (const char *)x + bytes <= g_pinned[i].p + g_pinned[i].bytes) return 1;
    return 0;
}

/* Large copies between pageable host memory and the device go through two pinned staging
 * buffers on a stream of their own: the CPU copy of chunk i+1 into (out of) one buffer overlaps
 * the DMA of chunk i from (into) the other.  A plain hipMemcpy from pageable memory stages through
 * the runtime's own small bounce buffers without that overlap and moved a batch-64 network input
 * (133 MB) several times slower. */
#define DN_STAGE_BYTES ((size_t)16 << 20)
#define DN_STAGE_MIN ((size_t)4 << 20)
static void *g_stage[2];
static hipEvent_t g_stage_ev[2];
static hipStream_t g_copy_stream;

/* memcpy between pageable and pinned memory, split over the host cores: one core moves ~8 GB/s,
 * less than the link, so a single-threaded copy would be the bottleneck of every large transfer */
void dn_host_copy(char *dst, const char *src, size_t bytes)
{
    const size_t piece = (size_t)1 << 20;
    const long pieces = (long)((bytes + piece - 1) / piece);
    long j;
#pragma omp parallel for schedule(static) num_threads(8) if (pieces >= 4)
    for (j = 0; j < pieces; ++j) {
        const size_t o = (size_t)j * piece;
        memcpy(dst + o, src + o, bytes - o < piece ? bytes - o : piece);
    }
}

static void staged_copy(char *dev, char *host, size_t bytes, int to_device)
{
    size_t off = 0, prev_off = 0, prev_len = 0;
    int i = 0, k;
    if (!g_stage[0]) {
        for (k = 0; k < 2; ++k) {
            hip_check_error(hipHostMalloc(&g_stage[k], DN_STAGE_BYTES, hipHostMallocDefault));
            hip_check_error(hipEventCreateWithFlags(&g_stage_ev[k], hipEventDisableTiming));
        }
        hip_check_error(hipStreamCreateWithFlags(&g_copy_stream, hipStreamNonBlocking));
    }
    /* everything queued so far has to be done before the copy stream touches the buffer */
    hip_check_error(hipStreamSynchronize(g_stream));
    for (; off < bytes; ++i) {
        const size_t len = bytes - off < DN_STAGE_BYTES ? bytes - off : DN_STAGE_BYTES;
        k = i & 1;
        if (to_device) {
            if (i >= 2) hip_check_error(hipEventSynchronize(g_stage_ev[k])); /* buffer k is free again */
            dn_host_copy((char *)g_stage[k], host + off, len);
            hip_check_error(hipMemcpyAsync(dev + off, g_stage[k], len, hipMemcpyHostToDevice, g_copy_stream));
            hip_check_error(hipEventRecord(g_stage_ev[k], g_copy_stream));
        } else {
            /* chunk i-2 left buffer k for the host before this loop came round again (see below) */
            hip_check_error(hipMemcpyAsync(g_stage[k], dev + off, len, hipMemcpyDeviceToHost, g_copy_stream));
            hip_check_error(hipEventRecord(g_stage_ev[k], g_copy_stream));
            if (i >= 1) { /* while chunk i is in flight, hand chunk i-1 to the caller */
                hip_check_error(hipEventSynchronize(g_stage_ev[k ^ 1]));
                dn_host_copy(host + prev_off, (const char *)g_stage[k ^ 1], prev_len);
            }
            prev_off = off;
            prev_len = len;
        }
        off += len;
    }
    hip_check_error(hipStreamSynchronize(g_copy_stream));
    if (!to_device && i >= 1) dn_host_copy(host + prev_off, (const char *)g_stage[(i - 1) & 1], prev_len);
}

/* The copies are synchronous, like the reference's cudaMemcpy (src/cuda.c:153-165); work
 * queued on a non-null stream is drained first so the copy sees it. */
void hip_push_array(float *x_gpu, float *x, size_t n)
{
    if (g_parse_only) return; /* the host copy is the only copy */
    if (g_npacked) packed_drop_range(x_gpu, n);
    if (sizeof(float) * n >= DN_STAGE_MIN && !dn_host_is_pinned(x, sizeof(float) * n)) {
        staged_copy((char *)x_gpu, (char *)x, sizeof(float) * n, 1);
        return;
    }
    if (g_stream) hip_check_error(hipStreamSynchronize(g_stream));
    hip_check_error(hipMemcpy(x_gpu, x, sizeof(float) * n, hipMemcpyHostToDevice));
}

void hip_pull_array(float *x_gpu, float *x, size_t n)
{
    if (g_parse_only) return;
    if (sizeof(float) * n >= DN_STAGE_MIN && !dn_host_is_pinned(x, sizeof(float) * n)) {
        staged_copy((char *)x_gpu, (char *)x, sizeof(float) * n, 0);
        return;
    }
    if (g_stream) hip_check_error(hipStreamSynchronize(g_stream));
    hip_check_error(hipMemcpy(x, x_gpu, sizeof(float) * n, hipMemcpyDeviceToHost));
}

void hip_push_int_array(int *x_gpu, int *x, size_t n)
{
    if (g_parse_only) return;
    if (g_stream) hip_check_error(hipStreamSynchronize(g_stream));
    hip_check_error(hipMemcpy(x_gpu, x, sizeof(int) * n, hipMemcpyHostToDevice));
}

void hip_pull_int_array(int *x_gpu, int *x, size_t n)
{
    if (g_parse_only) return;
    if (g_stream) hip_check_error(hipStreamSynchronize(g_stream));
    hip_check_error(hipMemcpy(x, x_gpu, sizeof(int) * n, hipMemcpyDeviceToHost));
}

float hip_mag_array(float *x_gpu, size_t n)
{
    float *tmp = (float *)calloc(n ? n : 1, sizeof(float));
    double sum = 0;
    size_t i;
    hip_pull_array(x_gpu, tmp, n);
    for (i = 0; i < n; ++i) sum += (double)tmp[i] * tmp[i];
    free(tmp);
    return (float)sqrt(sum);
}

float hip_compare(float *x_gpu, float *x, size_t n, char *s)
{
    float *tmp = (float *)calloc(n ? n : 1, sizeof(float));
    double err = 0;
    size_t i;
    hip_pull_array(x_gpu, tmp, n);
    for (i = 0; i < n; ++i) {
        double d = (double)tmp[i] - x[i];
        err += d * d;
    }
    free(tmp);
    printf("Error %s: %f\n", s, sqrt(err / (double)(n ? n : 1)));
    return (float)err;
}

void *hip_event_create(void)
{
    hipEvent_t ev;
    hip_check_error(hipEventCreate(&ev));
    return (void *)ev;
}

void hip_event_record(void *ev)
{
    hip_check_error(hipEventRecord((hipEvent_t)ev, g_stream));
}

float hip_event_elapsed_ms(void *start, void *stop)
{
    float ms = 0;
    hip_check_error(hipEventSynchronize((hipEvent_t)stop));
    hip_check_error(hipEventElapsedTime(&ms, (hipEvent_t)start, (hipEvent_t)stop));
    return ms;
}

void hip_event_destroy(void *ev)
{
    hip_check_error(hipEventDestroy((hipEvent_t)ev));
}

/* The reference's spellings, for objects compiled against its src/cuda.h. */
void cuda_set_device(int n) { hip_set_device(n); }
int cuda_get_device(void) { return hip_get_device(); }
float *cuda_make_array(float *x, size_t n) { return hip_make_array(x, n); }
int *cuda_make_int_array(int *x, size_t n) { return hip_make_int_array(x, n); }
void cuda_free(float *x_gpu) { hip_free(x_gpu); }
void cuda_push_array(float *x_gpu, float *x, size_t n) { hip_push_array(x_gpu, x, n); }
void cuda_pull_array(float *x_gpu, float *x, size_t n) { hip_pull_array(x_gpu, x, n); }
float cuda_mag_array(float *x_gpu, size_t n) { return hip_mag_array(x_gpu, n); }
float cuda_compare(float *x_gpu, float *x, size_t n, char *s) { return hip_compare(x_gpu, x, n, s); }
