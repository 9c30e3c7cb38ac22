/*
 * cfg_parser.c - builds a network from a cfg file: parse_network_cfg and the per-section
 * parsers of the layer types on the inference path.  Option names, defaults and the geometry
 * hand-over between consecutive layers follow the reference (src/parser.c:742-889 and the
 * parse_* functions cited below); hyper-parameters that only training reads are accepted and
 * ignored.  A section type outside this path ends the process with a message naming it.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "host.h"

typedef struct {
    int batch, inputs, h, w, c, index;
    network *net;
} size_params;

static const char *TRAINING_ONLY_NET_KEYS[] = {
    "learning_rate", "momentum", "decay", "notruth", "random", "adam", "B1", "B2", "eps", "max_crop",
    "min_crop", "max_ratio", "min_ratio", "center", "clip", "angle", "aspect", "saturation", "exposure",
    "hue", "policy", "burn_in", "power", "step", "scale", "steps", "scales", "gamma", "max_batches", 0};

static const char *PER_LAYER_KEYS[] = {"truth", "onlyforward", "stopbackward", "dontsave", "dontload",
                                       "numload", "dontloadscales", "learning_rate", "smooth", 0};

/* src/parser.c:47-85 */
static LAYER_TYPE section_type(const char *t)
{
    if (!strcmp(t, "[shortcut]")) return SHORTCUT;
    if (!strcmp(t, "[yolo]")) return YOLO;
    if (!strcmp(t, "[conv]") || !strcmp(t, "[convolutional]")) return CONVOLUTIONAL;
    if (!strcmp(t, "[net]") || !strcmp(t, "[network]")) return NETWORK;
    if (!strcmp(t, "[max]") || !strcmp(t, "[maxpool]")) return MAXPOOL;
    if (!strcmp(t, "[avg]") || !strcmp(t, "[avgpool]")) return AVGPOOL;
    if (!strcmp(t, "[soft]") || !strcmp(t, "[softmax]")) return SOFTMAX;
    if (!strcmp(t, "[route]")) return ROUTE;
    if (!strcmp(t, "[upsample]")) return UPSAMPLE;
    if (!strcmp(t, "[conn]") || !strcmp(t, "[connected]")) return CONNECTED;
    if (!strcmp(t, "[dropout]")) return DROPOUT;
    if (!strcmp(t, "[batchnorm]")) return BATCHNORM;
    if (!strcmp(t, "[reorg]")) return REORG;
    if (!strcmp(t, "[crop]")) return CROP;
    if (!strcmp(t, "[cost]")) return COST;
    if (!strcmp(t, "[region]")) return REGION;
    if (!strcmp(t, "[local]")) return LOCAL;
    if (!strcmp(t, "[detection]")) return DETECTION;
    return BLANK;
}

/* src/activations.c:44-63 */
ACTIVATION get_activation(char *s)
{
    static const char *names[] = {"logistic", "relu", "relie", "linear", "ramp", "tanh", "plse",
                                  "leaky", "elu", "loggy", "stair", "hardtan", "lhtan", "selu"};
    int i;
    for (i = 0; i < 14; ++i)
        if (strcmp(s, names[i]) == 0) return (ACTIVATION)i;
    fprintf(stderr, "Couldn't find activation function %s, going with ReLU\n", s);
    return RELU;
}

char *get_activation_string(ACTIVATION a)
{
    static char *names[] = {"logistic", "relu", "relie", "linear", "ramp", "tanh", "plse",
                            "leaky", "elu", "loggy", "stair", "hardtan", "lhtan", "selu"};
    if ((int)a < 0 || (int)a > 13) return "relu";
    return names[a];
}

/* src/network.c:110-175 */
char *get_layer_string(LAYER_TYPE a)
{
    switch (a) {
    case CONVOLUTIONAL: return "convolutional";
    case MAXPOOL: return "maxpool";
    case AVGPOOL: return "avgpool";
    case SOFTMAX: return "softmax";
    case ROUTE: return "route";
    case SHORTCUT: return "shortcut";
    case UPSAMPLE: return "upsample";
    case YOLO: return "yolo";
    case CONNECTED: return "connected";
    case DROPOUT: return "dropout";
    case BATCHNORM: return "batchnorm";
    case REORG: return "reorg";
    case CROP: return "crop";
    case COST: return "cost";
    case REGION: return "region";
    case LOCAL: return "local";
    case DETECTION: return "detection";
    default: return "none";
    }
}

static void need_image(size_params p, const char *what)
{
    if (!(p.h && p.w && p.c)) {
        char buf[128];
        snprintf(buf, sizeof buf, "Layer before %s layer must output image.", what);
        dn_fatal(buf);
    }
}

/* src/parser.c:179-207 */
static layer parse_convolutional(cfg_section *o, size_params p)
{
    int n = cfg_find_int(o, "filters", 1);
    int size = cfg_find_int(o, "size", 1);
    int stride = cfg_find_int(o, "stride", 1);
    int pad = cfg_find_int_quiet(o, "pad", 0);
    int padding = cfg_find_int_quiet(o, "padding", 0);
    int groups = cfg_find_int_quiet(o, "groups", 1);
    char *act;
    int bn, binary, xnor;
    layer l;
    if (pad) padding = size / 2;
    act = cfg_find_str(o, "activation", "logistic");
    need_image(p, "convolutional");
    bn = cfg_find_int_quiet(o, "batch_normalize", 0);
    binary = cfg_find_int_quiet(o, "binary", 0);
    xnor = cfg_find_int_quiet(o, "xnor", 0);
    l = make_convolutional_layer(p.batch, p.h, p.w, p.c, n, groups, size, stride, padding, get_activation(act),
                                 bn, binary, xnor, 0);
    l.flipped = cfg_find_int_quiet(o, "flipped", 0);
    (void)cfg_find_float_quiet(o, "dot", 0);
    return l;
}

/* src/parser.c:483-498 */
static layer parse_maxpool(cfg_section *o, size_params p)
{
    int stride = cfg_find_int(o, "stride", 1);
    int size = cfg_find_int(o, "size", stride);
    int padding = cfg_find_int_quiet(o, "padding", size - 1);
    need_image(p, "maxpool");
    return make_maxpool_layer(p.batch, p.h, p.w, p.c, size, stride, padding);
}

/* src/parser.c:500-511 */
static layer parse_avgpool(cfg_section *o, size_params p)
{
    (void)o;
    need_image(p, "avgpool");
    return make_avgpool_layer(p.batch, p.w, p.h, p.c);
}

/* src/parser.c:270-283 (tree and spatial modes are outside this path) */
static layer parse_softmax(cfg_section *o, size_params p)
{
    int groups = cfg_find_int_quiet(o, "groups", 1);
    layer l = make_softmax_layer(p.batch, p.inputs, groups);
    l.temperature = cfg_find_float_quiet(o, "temperature", 1);
    if (cfg_find_str(o, "tree", 0)) dn_fatal("softmax layer: tree= is not supported");
    l.w = p.w;
    l.h = p.h;
    l.c = p.c;
    if (cfg_find_float_quiet(o, "spatial", 0) != 0) dn_fatal("softmax layer: spatial= is not supported");
    l.noloss = cfg_find_int_quiet(o, "noloss", 0);
    return l;
}

/* src/parser.c:539-556 */
static layer parse_shortcut(cfg_section *o, size_params p, network *net)
{
    char *from = cfg_find(o, "from");
    int index;
    layer src, s;
    if (!from) dn_fatal("Shortcut layer must specify from");
    index = atoi(from);
    if (index < 0) index = p.index + index;
    if (index < 0 || index >= p.index) dn_fatal("Shortcut layer: from is out of range");
    src = net->layers[index];
    s = make_shortcut_layer(p.batch, index, p.w, p.h, p.c, src.out_w, src.out_h, src.out_c);
    s.activation = get_activation(cfg_find_str(o, "activation", "linear"));
    s.alpha = cfg_find_float_quiet(o, "alpha", 1);
    s.beta = cfg_find_float_quiet(o, "beta", 1);
    return s;
}

/* src/parser.c:592-599 */
static layer parse_upsample(cfg_section *o, size_params p)
{
    int stride = cfg_find_int(o, "stride", 2);
    layer l = make_upsample_layer(p.batch, p.w, p.h, p.c, stride);
    l.scale = cfg_find_float_quiet(o, "scale", 1);
    return l;
}

static int count_commas(const char *s)
{
    int n = 1;
    for (; *s; ++s)
        if (*s == ',') ++n;
    return n;
}

/* src/parser.c:601-640 */
static layer parse_route(cfg_section *o, size_params p, network *net)
{
    char *l = cfg_find(o, "layers");
    int n, i, *layers, *sizes;
    layer r, first;
    if (!l) dn_fatal("Route Layer must specify input layers");
    n = count_commas(l);
    layers = (int *)dn_calloc((size_t)n, sizeof(int));
    sizes = (int *)dn_calloc((size_t)n, sizeof(int));
    for (i = 0; i < n; ++i) {
        int index = atoi(l);
        char *next = strchr(l, ',');
        l = next ? next + 1 : l + strlen(l);
        if (index < 0) index = p.index + index;
        if (index < 0 || index >= p.index) dn_fatal("Route layer: input layer out of range");
        layers[i] = index;
        sizes[i] = net->layers[index].outputs;
    }
    first = net->layers[layers[0]];
    if (n == 1 && first.output_gpu) {
        /* one source: the reference copies it (src/route_layer.c:74-87); here the layer's output is a
         * view of the source's buffer - the same values, no launch, no second buffer */
        r = make_route_view(p.batch, layers[0], sizes[0], first.output_gpu);
        free(layers);
        free(sizes);
    } else {
        r = make_route_layer(p.batch, n, layers, sizes);
    }
    r.out_w = first.out_w;
    r.out_h = first.out_h;
    r.out_c = first.out_c;
    for (i = 1; i < n; ++i) {
        layer next = net->layers[layers[i]];
        if (next.out_w == first.out_w && next.out_h == first.out_h)
            r.out_c += next.out_c;
        else
            r.out_h = r.out_w = r.out_c = 0;
    }
    return r;
}

/* src/parser.c:259-268 */
static layer parse_connected(cfg_section *o, size_params p)
{
    int output = cfg_find_int(o, "output", 1);
    char *act = cfg_find_str(o, "activation", "logistic");
    int bn = cfg_find_int_quiet(o, "batch_normalize", 0);
    if (output < 1 || p.inputs < 1) dn_fatal("connected layer: needs inputs and output >= 1");
    return make_connected_layer(p.batch, p.inputs, output, get_activation(act), bn, 0);
}

/* src/parser.c:513-521; the caller aliases the output to the previous layer's (:829-836) */
static layer parse_dropout(cfg_section *o, size_params p)
{
    float probability = cfg_find_float(o, "probability", .5f);
    layer l = make_dropout_layer(p.batch, p.inputs, probability);
    l.out_w = p.w;
    l.out_h = p.h;
    l.out_c = p.c;
    return l;
}

/* src/parser.c:465-481 */
static layer parse_reorg(cfg_section *o, size_params p)
{
    int stride = cfg_find_int(o, "stride", 1);
    int reverse = cfg_find_int_quiet(o, "reverse", 0);
    int flatten = cfg_find_int_quiet(o, "flatten", 0);
    int extra = cfg_find_int_quiet(o, "extra", 0);
    need_image(p, "reorg");
    return make_reorg_layer(p.batch, p.w, p.h, p.c, stride, reverse, flatten, extra);
}

/* src/parser.c:441-463 */
static layer parse_crop(cfg_section *o, size_params p)
{
    int crop_height = cfg_find_int(o, "crop_height", 1);
    int crop_width = cfg_find_int(o, "crop_width", 1);
    int flip = cfg_find_int(o, "flip", 0);
    float angle = cfg_find_float(o, "angle", 0);
    float saturation = cfg_find_float(o, "saturation", 1);
    float exposure = cfg_find_float(o, "exposure", 1);
    int noadjust;
    layer l;
    need_image(p, "crop");
    noadjust = cfg_find_int_quiet(o, "noadjust", 0);
    l = make_crop_layer(p.batch, p.h, p.w, p.c, crop_height, crop_width, flip, angle, saturation, exposure);
    l.shift = cfg_find_float(o, "shift", 0);
    l.noadjust = noadjust;
    return l;
}

/* src/parser.c:429-439 */
static layer parse_cost(cfg_section *o, size_params p)
{
    float scale;
    (void)cfg_find_str(o, "type", "sse");
    scale = cfg_find_float_quiet(o, "scale", 1);
    (void)cfg_find_float_quiet(o, "ratio", 0);
    (void)cfg_find_float_quiet(o, "noobj", 1);
    (void)cfg_find_float_quiet(o, "thresh", 0);
    return make_cost_layer(p.batch, p.inputs, 0, scale);
}

/* src/parser.c:161-177: pad is the number of zero pixels itself here, not a flag */
static layer parse_local(cfg_section *o, size_params p)
{
    int n = cfg_find_int(o, "filters", 1);
    int size = cfg_find_int(o, "size", 1);
    int stride = cfg_find_int(o, "stride", 1);
    int pad = cfg_find_int(o, "pad", 0);
    ACTIVATION a = get_activation(cfg_find_str(o, "activation", "logistic"));
    need_image(p, "local");
    return make_local_layer(p.batch, p.h, p.w, p.c, n, size, stride, pad, a);
}

/* src/parser.c:405-428 */
static layer parse_detection(cfg_section *o, size_params p)
{
    static const char *training_keys[] = {"coord_scale", "forced", "object_scale", "noobject_scale", "class_scale",
                                          "jitter", "random", "reorg", 0};
    int coords = cfg_find_int(o, "coords", 1);
    int classes = cfg_find_int(o, "classes", 1);
    int rescore = cfg_find_int(o, "rescore", 0);
    int num = cfg_find_int(o, "num", 1);
    int side = cfg_find_int(o, "side", 7);
    int i;
    layer l = make_detection_layer(p.batch, p.inputs, num, side, classes, coords, rescore);
    l.softmax = cfg_find_int(o, "softmax", 0);
    l.sqrt = cfg_find_int(o, "sqrt", 0);
    l.max_boxes = cfg_find_int_quiet(o, "max", 90);
    for (i = 0; training_keys[i]; ++i) (void)cfg_find(o, training_keys[i]);
    return l;
}

/* src/parser.c:353-403 */
static layer parse_region(cfg_section *o, size_params p)
{
    static const char *training_keys[] = {"log", "sqrt", "max", "jitter", "rescore", "thresh", "classfix",
                                          "absolute", "random", "coord_scale", "object_scale", "noobject_scale",
                                          "mask_scale", "class_scale", "bias_match", 0};
    int coords = cfg_find_int(o, "coords", 4);
    int classes = cfg_find_int(o, "classes", 20);
    int num = cfg_find_int(o, "num", 1);
    char *a;
    int i;
    layer l = make_region_layer(p.batch, p.w, p.h, num, classes, coords);
    if (l.outputs != p.inputs) dn_fatal("region layer: the layer before it must output num*(classes+coords+1) channels");
    l.softmax = cfg_find_int(o, "softmax", 0);
    l.background = cfg_find_int_quiet(o, "background", 0);
    for (i = 0; training_keys[i]; ++i) (void)cfg_find(o, training_keys[i]);
    if (cfg_find_str(o, "tree", 0)) dn_fatal("region layer: tree= (hierarchical softmax) is not supported");
    if (cfg_find_str(o, "map", 0)) dn_fatal("region layer: map= is not supported");
    a = cfg_find_str(o, "anchors", 0);
    if (a) {
        int n = count_commas(a);
        for (i = 0; i < n && i < 2 * num; ++i) {
            char *next = strchr(a, ',');
            l.biases[i] = (float)atof(a);
            a = next ? next + 1 : a + strlen(a);
        }
    }
    return l;
}

/* src/parser.c:285-342 */
static layer parse_yolo(cfg_section *o, size_params p)
{
    int classes = cfg_find_int(o, "classes", 20);
    int total = cfg_find_int(o, "num", 1);
    int num = total;
    char *a = cfg_find_str(o, "mask", 0);
    int *mask = 0;
    layer l;
    if (a) {
        int n = count_commas(a), i;
        mask = (int *)dn_calloc((size_t)n, sizeof(int));
        for (i = 0; i < n; ++i) {
            char *next = strchr(a, ',');
            mask[i] = atoi(a);
            a = next ? next + 1 : a + strlen(a);
        }
        num = n;
    }
    l = make_yolo_layer(p.batch, p.w, p.h, num, total, mask, classes);
    if (l.outputs != p.inputs) dn_fatal("yolo layer: the layer before it must output n*(classes+5) channels");
    l.max_boxes = cfg_find_int_quiet(o, "max", 90);
    l.jitter = cfg_find_float(o, "jitter", .2f);
    l.ignore_thresh = cfg_find_float(o, "ignore_thresh", .5f);
    l.truth_thresh = cfg_find_float(o, "truth_thresh", 1);
    l.random = cfg_find_int_quiet(o, "random", 0);
    if (cfg_find_str(o, "map", 0)) dn_fatal("yolo layer: map= is not supported");
    a = cfg_find_str(o, "anchors", 0);
    if (a) {
        int n = count_commas(a), i;
        for (i = 0; i < n && i < 2 * total; ++i) {
            char *next = strchr(a, ',');
            l.biases[i] = (float)atof(a);
            a = next ? next + 1 : a + strlen(a);
        }
    }
    return l;
}

/* src/parser.c:655-679: batch is divided by subdivisions and fixed here for the network's life */
static void parse_net_options(cfg_section *o, network *net)
{
    int subdivs, i;
    net->batch = cfg_find_int(o, "batch", 1);
    subdivs = cfg_find_int(o, "subdivisions", 1);
    net->time_steps = cfg_find_int_quiet(o, "time_steps", 1);
    if (subdivs < 1) subdivs = 1;
    net->batch /= subdivs;
    net->batch *= net->time_steps;
    net->subdivisions = subdivs;
    net->h = cfg_find_int_quiet(o, "height", 0);
    net->w = cfg_find_int_quiet(o, "width", 0);
    net->c = cfg_find_int_quiet(o, "channels", 0);
    net->inputs = cfg_find_int_quiet(o, "inputs", net->h * net->w * net->c);
    if (!net->inputs && !(net->h && net->w && net->c)) dn_fatal("No input parameters supplied");
    if (net->batch < 1) dn_fatal("batch/subdivisions must be at least 1");
    for (i = 0; TRAINING_ONLY_NET_KEYS[i]; ++i) (void)cfg_find(o, TRAINING_ONLY_NET_KEYS[i]);
}

network *parse_network_cfg(char *filename)
{
    cfg_file *f = cfg_read(filename);
    network *net;
    size_params p;
    int count, i;
    if (f->n < 1) dn_fatal("Config file has no sections");
    if (section_type(f->sections[0].type) != NETWORK) dn_fatal("First section must be [net] or [network]");
    net = make_network(f->n - 1);
    net->gpu_index = gpu_index;
    if (gpu_index < 0) dn_fatal("this library has no CPU path: gpu_index must name a device");
    hip_set_device(gpu_index);
    parse_net_options(&f->sections[0], net);
    cfg_report_unused(&f->sections[0]);
    p.h = net->h;
    p.w = net->w;
    p.c = net->c;
    p.inputs = net->inputs;
    p.batch = net->batch;
    p.net = net;
    if (dn_verbose) fprintf(stderr, "layer     filters    size              input                output\n");
    for (count = 0; count < net->n; ++count) {
        cfg_section *o = &f->sections[count + 1];
        LAYER_TYPE lt = section_type(o->type);
        layer l;
        p.index = count;
        if (dn_verbose) fprintf(stderr, "%5d ", count);
        switch (lt) {
        case CONVOLUTIONAL: l = parse_convolutional(o, p); break;
        case MAXPOOL: l = parse_maxpool(o, p); break;
        case AVGPOOL: l = parse_avgpool(o, p); break;
        case SOFTMAX: l = parse_softmax(o, p); break;
        case ROUTE: l = parse_route(o, p, net); break;
        case UPSAMPLE: l = parse_upsample(o, p); break;
        case SHORTCUT: l = parse_shortcut(o, p, net); break;
        case YOLO: l = parse_yolo(o, p); break;
        case CONNECTED: l = parse_connected(o, p); break;
        case REORG: l = parse_reorg(o, p); break;
        case CROP: l = parse_crop(o, p); break;
        case COST: l = parse_cost(o, p); break;
        case REGION: l = parse_region(o, p); break;
        case LOCAL: l = parse_local(o, p); break;
        case DETECTION: l = parse_detection(o, p); break;
        case BATCHNORM: l = make_batchnorm_layer(p.batch, p.w, p.h, p.c); break; /* src/parser.c:533-537 */
        case DROPOUT:
            if (count == 0) dn_fatal("dropout cannot be the first layer");
            l = parse_dropout(o, p);
            l.output = net->layers[count - 1].output;
            l.output_gpu = net->layers[count - 1].output_gpu;
            break;
        default: {
            char buf[256];
            snprintf(buf, sizeof buf, "layer type %s (section %d) is outside the convolution forward path this "
                     "library implements", o->type, count);
            dn_fatal(buf);
            memset(&l, 0, sizeof l);
        }
        }
        l.truth = cfg_find_int_quiet(o, "truth", 0);
        l.onlyforward = cfg_find_int_quiet(o, "onlyforward", 0);
        l.dontload = cfg_find_int_quiet(o, "dontload", 0);
        l.numload = cfg_find_int_quiet(o, "numload", 0);
        l.dontloadscales = cfg_find_int_quiet(o, "dontloadscales", 0);
        for (i = 0; PER_LAYER_KEYS[i]; ++i) (void)cfg_find(o, PER_LAYER_KEYS[i]);
        cfg_report_unused(o);
        net->layers[count] = l;
        p.h = l.out_h;
        p.w = l.out_w;
        p.c = l.out_c;
        p.inputs = l.outputs;
    }
    cfg_free(f);
    {
        /* the output layer is the last one that is not a cost layer (src/network.c:689-697); the
         * host sees its output after every forward (src/network.c:786) */
        layer *last = &net->layers[net->n - 1];
        layer *out = last;
        for (i = net->n - 1; i >= 0; --i)
            if (net->layers[i].type != COST) break;
        if (i < 0) dn_fatal("network has no layers besides cost layers");
        out = &net->layers[i];
        net->outputs = out->outputs;
        net->truths = out->outputs;
        if (last->truths) net->truths = last->truths;
        if (!out->output) {
            /* a dropout layer's buffers are those of the layer before it (src/parser.c:829-836): the
             * host copy belongs to that owner, which free_layer releases, and every dropout layer
             * behind the owner shares it */
            int owner = i, j;
            while (owner > 0 && net->layers[owner].type == DROPOUT) --owner;
            net->layers[owner].output = hip_host_alloc((size_t)out->outputs * out->batch);
            for (j = owner + 1; j < net->n && net->layers[j].type == DROPOUT; ++j)
                net->layers[j].output = net->layers[owner].output;
        }
        net->output = out->output;
        net->output_gpu = out->output_gpu;
    }
    net->max_batch = net->batch;
    net->input = (float *)dn_calloc((size_t)net->inputs * net->batch, sizeof(float));
    net->input_gpu = hip_make_array(net->input, (size_t)net->inputs * net->batch);
    return net;
}
