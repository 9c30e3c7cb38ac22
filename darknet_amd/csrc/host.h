/*
 * host.h - declarations shared by the host-side C files (cfg reader, layer constructors,
 * network runtime, weights I/O).  Not installed; the public API is include/darknet_amd.h.
 */
#ifndef DN_HOST_H
#define DN_HOST_H

#include "darknet_amd.h"
#include "hip.h"

/* One `[section]` of a cfg file with its key=value lines in file order. */
typedef struct {
    char *key;
    char *val;
    int used;
} cfg_option;

typedef struct {
    char *type;          /* the header line with blanks removed, e.g. "[convolutional]" */
    cfg_option *opts;
    int nopts, cap;
} cfg_section;

typedef struct {
    cfg_section *sections;
    int n, cap;
} cfg_file;

cfg_file *cfg_read(const char *filename);
void cfg_free(cfg_file *f);
char *cfg_find(cfg_section *s, const char *key);
char *cfg_find_str(cfg_section *s, const char *key, char *def);
int cfg_find_int(cfg_section *s, const char *key, int def);
int cfg_find_int_quiet(cfg_section *s, const char *key, int def);
float cfg_find_float(cfg_section *s, const char *key, float def);
float cfg_find_float_quiet(cfg_section *s, const char *key, float def);
void cfg_report_unused(cfg_section *s);

layer make_route_view(int batch, int input_layer, int input_size, float *source_output_gpu);

void dn_forward_gated(network *net, int gate_layer, void (*gate)(void *), void *gate_arg);
void dn_pipeline_free(network *net);

extern int dn_verbose;
void *dn_calloc(size_t n, size_t size);

#endif
