/*
 * cfg_reader.c - reads darknet's cfg grammar into sections of key=value options.
 *
 * Grammar, as the reference implements it (src/parser.c:891-924 read_cfg,
 * src/option_list.c:52-77 read_option, src/utils.c:302-313 strip, :335-364 fgetl):
 *   - every blank, tab and newline is removed from a line before anything else;
 *   - a line starting with '[' opens a section, its whole text is the section type;
 *   - empty lines and lines starting with '#' or ';' are skipped;
 *   - any other line is split at the first '='; a line whose only '=' is its last
 *     character is reported and dropped;
 *   - lookups return the first option with a matching key and mark it used; numeric values go
 *     through atoi / atof; the non-quiet finders print the default they fall back to.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "host.h"

void *dn_calloc(size_t n, size_t size)
{
    void *p = calloc(n ? n : 1, size ? size : 1);
    if (!p) dn_fatal("Malloc error");
    return p;
}

static char *read_line(FILE *fp)
{
    size_t cap = 256, len = 0;
    char *buf;
    int ch;
    if (feof(fp)) return 0;
    buf = (char *)malloc(cap);
    if (!buf) dn_fatal("Malloc error");
    while ((ch = fgetc(fp)) != EOF && ch != '\n') {
        if (len + 2 > cap) {
            cap *= 2;
            buf = (char *)realloc(buf, cap);
            if (!buf) dn_fatal("Malloc error");
        }
        buf[len++] = (char)ch;
    }
    if (ch == EOF && len == 0) {
        free(buf);
        return 0;
    }
    buf[len] = 0;
    return buf;
}

static void squeeze(char *s)
{
    char *dst = s;
    for (; *s; ++s)
        if (*s != ' ' && *s != '\t' && *s != '\n') *dst++ = *s;
    *dst = 0;
}

static cfg_section *add_section(cfg_file *f, char *type)
{
    cfg_section *s;
    if (f->n == f->cap) {
        f->cap = f->cap ? f->cap * 2 : 32;
        f->sections = (cfg_section *)realloc(f->sections, sizeof(cfg_section) * (size_t)f->cap);
        if (!f->sections) dn_fatal("Malloc error");
    }
    s = &f->sections[f->n++];
    memset(s, 0, sizeof *s);
    s->type = type;
    return s;
}

static void add_option(cfg_section *s, char *key, char *val)
{
    if (s->nopts == s->cap) {
        s->cap = s->cap ? s->cap * 2 : 8;
        s->opts = (cfg_option *)realloc(s->opts, sizeof(cfg_option) * (size_t)s->cap);
        if (!s->opts) dn_fatal("Malloc error");
    }
    s->opts[s->nopts].key = key;
    s->opts[s->nopts].val = val;
    s->opts[s->nopts].used = 0;
    s->nopts++;
}

cfg_file *cfg_read(const char *filename)
{
    FILE *fp = fopen(filename, "r");
    cfg_file *f;
    cfg_section *cur = 0;
    char *line;
    int nu = 0;
    if (!fp) {
        /* file_error of the reference (src/utils.c:281-285) */
        fprintf(stderr, "Couldn't open file: %s\n", filename);
        exit(0);
    }
    f = (cfg_file *)dn_calloc(1, sizeof *f);
    while ((line = read_line(fp)) != 0) {
        ++nu;
        squeeze(line);
        switch (line[0]) {
        case '[':
            cur = add_section(f, line);
            break;
        case '\0':
        case '#':
        case ';':
            free(line);
            break;
        default: {
            char *eq = strchr(line, '=');
            size_t len = strlen(line);
            if (!cur || (eq && (size_t)(eq - line) == len - 1)) {
                fprintf(stderr, "Config file error line %d, could parse: %s\n", nu, line);
                free(line);
                break;
            }
            if (eq) {
                *eq = 0;
                add_option(cur, line, eq + 1);
            } else {
                add_option(cur, line, 0);
            }
        }
        }
    }
    fclose(fp);
    return f;
}

void cfg_free(cfg_file *f)
{
    int i, j;
    if (!f) return;
    for (i = 0; i < f->n; ++i) {
        for (j = 0; j < f->sections[i].nopts; ++j) free(f->sections[i].opts[j].key);
        free(f->sections[i].opts);
        free(f->sections[i].type);
    }
    free(f->sections);
    free(f);
}

char *cfg_find(cfg_section *s, const char *key)
{
    int i;
    for (i = 0; i < s->nopts; ++i)
        if (strcmp(s->opts[i].key, key) == 0) {
            s->opts[i].used = 1;
            return s->opts[i].val;
        }
    return 0;
}

char *cfg_find_str(cfg_section *s, const char *key, char *def)
{
    char *v = cfg_find(s, key);
    if (v) return v;
    if (def && dn_verbose) fprintf(stderr, "%s: Using default '%s'\n", key, def);
    return def;
}

int cfg_find_int(cfg_section *s, const char *key, int def)
{
    char *v = cfg_find(s, key);
    if (v) return atoi(v);
    if (dn_verbose) fprintf(stderr, "%s: Using default '%d'\n", key, def);
    return def;
}

int cfg_find_int_quiet(cfg_section *s, const char *key, int def)
{
    char *v = cfg_find(s, key);
    return v ? atoi(v) : def;
}

float cfg_find_float(cfg_section *s, const char *key, float def)
{
    char *v = cfg_find(s, key);
    if (v) return (float)atof(v);
    if (dn_verbose) fprintf(stderr, "%s: Using default '%lf'\n", key, def);
    return def;
}

float cfg_find_float_quiet(cfg_section *s, const char *key, float def)
{
    char *v = cfg_find(s, key);
    return v ? (float)atof(v) : def;
}

void cfg_report_unused(cfg_section *s)
{
    int i;
    if (!dn_verbose) return;
    for (i = 0; i < s->nopts; ++i)
        if (!s->opts[i].used) fprintf(stderr, "Unused field: '%s = %s'\n", s->opts[i].key, s->opts[i].val);
}
