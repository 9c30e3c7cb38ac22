/*
 * pipeline.c - network_predict in two halves, so that the copies of consecutive batches overlap
 * the compute of the batch between them.
 *
 * network_predict (src/network.c:497-508 of the reference, with the synchronous cudaMemcpy of
 * :766 and :786 and of src/yolo_layer.c:360) is upload, compute, download one after the other;
 * at batch 64 of yolov3-416 the two copies (133 MB in, 232 MB out) take as long as the compute.
 * Here a batch is submitted and collected separately, with up to two batches in flight:
 *
 *   submit(n)   host: the input is taken into pinned memory (a pinned input is used where it is)
 *               upload stream:   H2D into input slot n%2                    -> event uploaded[n%2]
 *               launch stream:   waits uploaded, runs the layer loop        -> event computed[n%2]
 *                                (before the first layer that writes a buffer the host reads, it
 *                                also waits for downloaded[(n-1)%2]: the previous batch's outputs
 *                                must have left those buffers)
 *               download stream: waits computed, D2H of the yolo heads and the output layer into
 *                                host slot n%2                              -> event downloaded[n%2]
 *   collect()   host: waits downloaded of the oldest batch in flight, hands out host slot
 *
 * The three streams are at the default priority; the upload and download streams are non-blocking
 * streams of their own, so H2D of batch n+1 and D2H of batch n-1 run on the two copy engines while
 * batch n computes.  The kernels, their arguments and their order are those of network_predict:
 * the outputs are the same bits.
 */
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>

#include <stdlib.h>
#include <string.h>

#include "host.h"

#define DN_PIPE_SLOTS 2
#define DN_PIPE_MAX_PULLED 16

typedef struct {
    int npulled;
    int pulled[DN_PIPE_MAX_PULLED];          /* layers whose output the host reads: yolo heads, output layer */
    int first_pulled;                        /* the earliest of them */
    size_t input_floats;                     /* capacity of an input slot (cfg batch) */
    float *input_gpu[DN_PIPE_SLOTS];         /* slot 0 is the network's own input buffer */
    float *input_stage[DN_PIPE_SLOTS];       /* pinned */
    float *out_host[DN_PIPE_SLOTS][DN_PIPE_MAX_PULLED]; /* pinned */
    hipStream_t upload, download;
    hipEvent_t uploaded[DN_PIPE_SLOTS], computed[DN_PIPE_SLOTS], downloaded[DN_PIPE_SLOTS];
    int submitted, collected;                /* batches submitted / collected so far */
    int last_slot;                           /* slot of the batch collected last, -1 before the first */
} pipeline;

/* network.c: the layer loop with a callback in front of the first layer at or after `layer` */
void dn_forward_gated(network *net, int layer, void (*gate)(void *), void *arg);

static void pipe_check(hipError_t e) { hip_check_error((int)e); }

static pipeline *pipe_of(network *net)
{
    pipeline *p = (pipeline *)net->pipeline;
    int i, s;
    const int cap = net->max_batch > net->batch ? net->max_batch : net->batch;
    if (p) return p;
    hip_require_device("network_predict_submit");
    p = (pipeline *)dn_calloc(1, sizeof(pipeline));
    p->last_slot = -1;
    p->first_pulled = net->n;
    for (i = 0; i < net->n; ++i)   /* what network_pull_outputs pulls: the yolo heads, then the output layer */
        if (net->layers[i].type == YOLO && net->layers[i].output_gpu && i < net->n - 1) {
            if (p->npulled == DN_PIPE_MAX_PULLED - 1) dn_fatal("network_predict_submit: too many yolo heads");
            p->pulled[p->npulled++] = i;
        }
    for (i = net->n - 1; i > 0 && net->layers[i].type == COST; --i) {}
    if (!net->layers[i].output_gpu) dn_fatal("network_predict_submit: the output layer has no device buffer");
    p->pulled[p->npulled++] = i;
    for (i = 0; i < p->npulled; ++i)
        if (p->pulled[i] < p->first_pulled) p->first_pulled = p->pulled[i];
    p->input_floats = (size_t)net->inputs * cap;
    p->input_gpu[0] = net->input_gpu;
    p->input_gpu[1] = hip_make_array(0, p->input_floats);
    for (s = 0; s < DN_PIPE_SLOTS; ++s) {
        p->input_stage[s] = hip_host_alloc(p->input_floats);
        for (i = 0; i < p->npulled; ++i)
            p->out_host[s][i] = hip_host_alloc((size_t)net->layers[p->pulled[i]].outputs * cap);
        pipe_check(hipEventCreateWithFlags(&p->uploaded[s], hipEventDisableTiming));
        pipe_check(hipEventCreateWithFlags(&p->computed[s], hipEventDisableTiming));
        pipe_check(hipEventCreateWithFlags(&p->downloaded[s], hipEventDisableTiming));
    }
    pipe_check(hipStreamCreateWithFlags(&p->upload, hipStreamNonBlocking));
    pipe_check(hipStreamCreateWithFlags(&p->download, hipStreamNonBlocking));
    net->pipeline = p;
    return p;
}

void dn_pipeline_free(network *net)
{
    pipeline *p = (pipeline *)net->pipeline;
    int i, s;
    if (!p) return;
    pipe_check(hipStreamSynchronize(p->upload));
    pipe_check(hipStreamSynchronize(p->download));
    hip_synchronize();
    hip_free(p->input_gpu[1]);
    for (s = 0; s < DN_PIPE_SLOTS; ++s) {
        hip_host_free(p->input_stage[s]);
        for (i = 0; i < p->npulled; ++i) hip_host_free(p->out_host[s][i]);
        pipe_check(hipEventDestroy(p->uploaded[s]));
        pipe_check(hipEventDestroy(p->computed[s]));
        pipe_check(hipEventDestroy(p->downloaded[s]));
    }
    pipe_check(hipStreamDestroy(p->upload));
    pipe_check(hipStreamDestroy(p->download));
    free(p);
    net->pipeline = 0;
}

typedef struct {
    hipStream_t stream;
    hipEvent_t event;
} gate_arg;

static void wait_for_previous_download(void *arg)
{
    gate_arg *g = (gate_arg *)arg;
    pipe_check(hipStreamWaitEvent(g->stream, g->event, 0));
}

void network_predict_submit(network *net, float *input)
{
    pipeline *p = pipe_of(net);
    const int slot = p->submitted % DN_PIPE_SLOTS;
    const size_t in_bytes = sizeof(float) * (size_t)net->inputs * net->batch;
    hipStream_t launch = (hipStream_t)hip_get_stream();
    float *own_input = net->input_gpu;
    gate_arg gate;
    const float *src = input;
    int i;
    if (p->submitted - p->collected >= DN_PIPE_SLOTS)
        dn_fatal("network_predict_submit: two batches are in flight already; collect one first");
    if ((size_t)net->inputs * net->batch > p->input_floats)
        dn_fatal("network_predict_submit: the batch grew beyond the one the buffers were made for");
    hip_set_device(net->gpu_index);

    /* the slot's staging buffer and device input were last used by batch n-2, collected by now */
    if (!dn_host_is_pinned(input, in_bytes)) {
        dn_host_copy((char *)p->input_stage[slot], (const char *)input, in_bytes);
        src = p->input_stage[slot];
    }
    pipe_check(hipMemcpyAsync(p->input_gpu[slot], src, in_bytes, hipMemcpyHostToDevice, p->upload));
    pipe_check(hipEventRecord(p->uploaded[slot], p->upload));

    pipe_check(hipStreamWaitEvent(launch, p->uploaded[slot], 0));
    gate.stream = launch;
    gate.event = p->downloaded[slot ^ 1];
    net->input_gpu = p->input_gpu[slot];
    /* the previous batch (if any is still on its way out) must have left the buffers the host reads
     * before this batch writes them; everything in front of that layer overlaps its download */
    dn_forward_gated(net, p->submitted > p->collected ? p->first_pulled : -1, wait_for_previous_download, &gate);
    net->input_gpu = own_input;
    pipe_check(hipEventRecord(p->computed[slot], launch));

    pipe_check(hipStreamWaitEvent(p->download, p->computed[slot], 0));
    for (i = 0; i < p->npulled; ++i) {
        const layer *l = &net->layers[p->pulled[i]];
        pipe_check(hipMemcpyAsync(p->out_host[slot][i], l->output_gpu, sizeof(float) * (size_t)l->outputs * l->batch,
                                  hipMemcpyDeviceToHost, p->download));
    }
    pipe_check(hipEventRecord(p->downloaded[slot], p->download));
    ++p->submitted;
}

float *network_predict_collect(network *net)
{
    pipeline *p = (pipeline *)net->pipeline;
    int slot;
    if (!p || p->collected >= p->submitted) dn_fatal("network_predict_collect: no batch is in flight");
    slot = p->collected % DN_PIPE_SLOTS;
    pipe_check(hipEventSynchronize(p->downloaded[slot]));
    ++p->collected;
    p->last_slot = slot;
    return p->out_host[slot][p->npulled - 1];
}

float *network_collected_output(network *net, int layer_index)
{
    pipeline *p = (pipeline *)net->pipeline;
    int i;
    if (!p || p->last_slot < 0) dn_fatal("network_collected_output: nothing has been collected yet");
    for (i = 0; i < p->npulled; ++i)
        if (p->pulled[i] == layer_index) return p->out_host[p->last_slot][i];
    dn_fatal("network_collected_output: the host reads only the yolo heads and the output layer");
    return 0;
}

int network_predict_in_flight(network *net)
{
    pipeline *p = (pipeline *)net->pipeline;
    return p ? p->submitted - p->collected : 0;
}
