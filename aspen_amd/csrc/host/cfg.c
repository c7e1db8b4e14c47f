/*
 * cfg.c -- Darknet-style model description reader.
 *
 * Accepts the dialect the reference reads (section names: reference src/darknet_parser.c:410-436,
 * keys: :460-486, activation names: :393-408) and derives each layer's input/output geometry the
 * way the reference does (reference src/input_parser.c:35-127).  `batch_normalize=` is ignored, as
 * in the reference: batch norm only arrives through the weight file.
 */
#include <ctype.h>
#include "internal.h"

#define MAX_OPTS 32
typedef struct { char key[48]; char val[160]; } opt_t;
typedef struct { char name[48]; opt_t opts[MAX_OPTS]; int num_opts; } section_t;

static LAYER_TYPE section_type (const char *s)
{
    static const struct { const char *name; LAYER_TYPE type; } tab[] = {
        {"[net]", INPUT_LAYER}, {"[network]", INPUT_LAYER}, {"[conv]", CONV_LAYER}, {"[convolutional]", CONV_LAYER},
        {"[shortcut]", RESIDUAL_LAYER}, {"[max]", MAXPOOL_LAYER}, {"[maxpool]", MAXPOOL_LAYER},
        {"[avg]", AVGPOOL_LAYER}, {"[avgpool]", AVGPOOL_LAYER}, {"[conn]", FC_LAYER}, {"[connected]", FC_LAYER},
        {"[soft]", SOFTMAX_LAYER}, {"[softmax]", SOFTMAX_LAYER}, {"[matmul]", MATMUL_LAYER},
        {"[attention_k]", K_ATTENTION_LAYER}, {"[attention_v]", V_ATTENTION_LAYER}, {"[layernorm]", LAYERNORM_LAYER},
        {"[yolo]", YOLO_LAYER}, {"[append]", APPEND_LAYER},
    };
    for (size_t i = 0; i < sizeof (tab) / sizeof (tab[0]); i++)
        if (strcmp (s, tab[i].name) == 0) return tab[i].type;
    return NO_LAYER_TYPE;
}

static LAYER_ACT activation_type (const char *s)
{
    if (s == NULL) return NO_ACTIVATION;
    static const struct { const char *name; LAYER_ACT act; } tab[] = {
        {"logistic", SIGMOID}, {"linear", NO_ACTIVATION}, {"none", NO_ACTIVATION}, {"leaky", LEAKY_RELU},
        {"relu", RELU}, {"elu", ELU}, {"selu", SELU}, {"tanh", TANH}, {"gelu", GELU}, {"gelu_acc", GELU_ACCURATE},
    };
    for (size_t i = 0; i < sizeof (tab) / sizeof (tab[0]); i++)
        if (strcmp (s, tab[i].name) == 0) return tab[i].act;
    ERROR_PRTF ("Couldn't find activation function %s, going with ReLU\n", s);
    return RELU;
}

static const char *opt_str (const section_t *s, const char *key)
{
    for (int i = 0; i < s->num_opts; i++)
        if (strcmp (s->opts[i].key, key) == 0) return s->opts[i].val;
    return NULL;
}
static int opt_int (const section_t *s, const char *key, int def)
{
    const char *v = opt_str (s, key);
    return v ? atoi (v) : def;
}

static char *trim (char *s)
{
    while (*s && isspace ((unsigned char)*s)) s++;
    char *e = s + strlen (s);
    while (e > s && isspace ((unsigned char)e[-1])) *--e = 0;
    return s;
}

static section_t *read_sections (const char *path, int *count)
{
    FILE *fp = fopen (path, "r");
    if (fp == NULL) { ERROR_PRTF ("Couldn't open cfg file %s\n", path); return NULL; }
    int cap = 64, n = 0, skipping = 0;
    section_t *secs = calloc (cap, sizeof (section_t));
    if (secs == NULL) { ERROR_PRTF ("Out of host memory reading %s\n", path); fclose (fp); return NULL; }
    char line[512];
    while (fgets (line, sizeof (line), fp))
    {
        char *p = trim (line);
        if (*p == 0 || *p == '#' || *p == ';') continue;
        if (*p == '[')
        {
            if (section_type (p) == NO_LAYER_TYPE) { ERROR_PRTF ("Unsupported section type: %s\n", p); skipping = 1; continue; }
            skipping = 0;
            if (n == cap)
            {
                section_t *grown = realloc (secs, 2 * (size_t)cap * sizeof (section_t));
                if (grown == NULL) { ERROR_PRTF ("Out of host memory reading %s\n", path); free (secs); fclose (fp); return NULL; }
                secs = grown; cap *= 2;
                memset (secs + n, 0, (size_t)(cap - n) * sizeof (section_t));
            }
            strncpy (secs[n].name, p, sizeof (secs[n].name) - 1);
            n++;
            continue;
        }
        char *eq = strchr (p, '=');
        if (eq == NULL || n == 0 || skipping) continue;
        *eq = 0;
        section_t *s = &secs[n - 1];
        if (s->num_opts == MAX_OPTS) continue;
        strncpy (s->opts[s->num_opts].key, trim (p), sizeof (s->opts[0].key) - 1);
        strncpy (s->opts[s->num_opts].val, trim (eq + 1), sizeof (s->opts[0].val) - 1);
        s->num_opts++;
    }
    fclose (fp);
    *count = n;
    return secs;
}

static int conv_out (unsigned int in, unsigned int pad, unsigned int dil, unsigned int k, unsigned int stride)
{
    return (int)(in + 2 * pad - dil * (k - 1) - 1) / (int)stride + 1;
}

/* number list "a, b,  c" -> up to max values; returns the count */
static int parse_numbers (const char *str, float *dst, int max)
{
    int n = 0;
    while (str && *str && n < max)
    {
        char *end;
        const float v = strtof (str, &end);
        if (end == str) break;
        dst[n++] = v;
        str = end;
        while (*str == ',' || isspace ((unsigned char)*str)) str++;
    }
    return n;
}

/* [yolo]: rows = classes + 5; the layer's three anchor boxes are picked from `anchors` by `mask`
   (reference src/darknet_parser.c:487-545) */
static int parse_yolo (const section_t *s, aspen_layer_t *L)
{
    float mask[16], anchors[64];
    const int nm = parse_numbers (opt_str (s, "mask"), mask, 16), na = parse_numbers (opt_str (s, "anchors"), anchors, 64);
    if (nm < 3) { ERROR_PRTF ("YOLO layer has no mask.\n"); return -1; }
    if (na < 2) { ERROR_PRTF ("YOLO layer has no anchors.\n"); return -1; }
    L->params[OUT_C] = (unsigned int)opt_int (s, "classes", 0) + 5;
    for (int i = 0; i < 3; i++)
    {
        const int m = (int)mask[i];
        if (m < 0 || 2 * m + 1 >= na) { ERROR_PRTF ("YOLO layer: mask %d has no anchor.\n", m); return -1; }
        L->anchors[2 * i] = anchors[2 * m]; L->anchors[2 * i + 1] = anchors[2 * m + 1];
    }
    return 0;
}

/* in/out geometry of one layer from its parent (reference src/input_parser.c:35-127) */
static int set_inout (aspen_dnn_t *dnn, aspen_layer_t *L)
{
    unsigned int *p = L->params;
    if (L->type == INPUT_LAYER)
    {
        if (p[MAT_M] != 0) { p[OUT_H] = 1; p[OUT_W] = p[MAT_N]; p[OUT_C] = p[MAT_M]; }
        else { p[OUT_C] = p[IN_C]; p[OUT_H] = p[IN_H]; p[OUT_W] = p[IN_W]; }
        return 0;
    }
    const aspen_layer_t *P = &dnn->layers[L->parent_idx[PARENT_0]];
    p[IN_H] = P->params[OUT_H]; p[IN_W] = P->params[OUT_W]; p[IN_C] = P->params[OUT_C];
    switch (L->type)
    {
    case CONV_LAYER: case MAXPOOL_LAYER: case AVGPOOL_LAYER:
        if (p[STRIDE] == 0) p[STRIDE] = 1;
        if (p[DILATION] == 0) p[DILATION] = 1;
        if (p[DILATION] != 1) { ERROR_PRTF ("layer %u: dilation %u is not supported\n", L->layer_idx, p[DILATION]); return -1; }
        if (p[WEIGHT_H] == 0) { ERROR_PRTF ("layer %u: missing size=\n", L->layer_idx); return -1; }
        p[OUT_H] = conv_out (p[IN_H], p[PADDING], p[DILATION], p[WEIGHT_H], p[STRIDE]);
        p[OUT_W] = conv_out (p[IN_W], p[PADDING], p[DILATION], p[WEIGHT_W], p[STRIDE]);
        if (L->type != CONV_LAYER) p[OUT_C] = p[IN_C];
        if ((int)p[OUT_H] < 1 || (int)p[OUT_W] < 1 || p[OUT_C] == 0) { ERROR_PRTF ("layer %u: empty output\n", L->layer_idx); return -1; }
        return 0;
    case FC_LAYER:
        p[OUT_H] = 1; p[OUT_W] = 1;
        return 0;
    case SOFTMAX_LAYER:
        p[OUT_H] = 1; p[OUT_W] = 1; p[OUT_C] = p[IN_C];
        return 0;
    case RESIDUAL_LAYER:
        if (p[MAT_M] != 0) { p[OUT_H] = 1; p[OUT_W] = p[MAT_N]; p[OUT_C] = p[MAT_M]; }
        else { p[OUT_C] = p[IN_C]; p[OUT_H] = p[IN_H]; p[OUT_W] = p[IN_W]; }
        if (L->parent_idx[PARENT_1] < 0) { ERROR_PRTF ("layer %u: shortcut without from=\n", L->layer_idx); return -1; }
        return 0;
    case MATMUL_LAYER:
        p[MAT_K] = P->params[MAT_M];
        if (p[MAT_K] == 0 || p[MAT_M] == 0) { ERROR_PRTF ("layer %u: matmul needs M= and a matrix parent\n", L->layer_idx); return -1; }
        return 0;
    case LAYERNORM_LAYER: case V_ATTENTION_LAYER:
        if (L->type == V_ATTENTION_LAYER && (L->parent_idx[PARENT_1] < 0 || p[NUM_HEAD] == 0)) { ERROR_PRTF ("layer %u: attention_v needs from= and n_head=\n", L->layer_idx); return -1; }
        return 0;
    case YOLO_LAYER:
        if (p[STRIDE] == 0) p[STRIDE] = 1;
        if (p[OUT_C] < 5 || p[IN_C] % p[OUT_C] != 0 || p[IN_C] / p[OUT_C] > 3)
        { ERROR_PRTF ("layer %u: yolo needs (classes + 5) x (at most 3 anchors) input channels, got %u for %u rows\n", L->layer_idx, p[IN_C], p[OUT_C]); return -1; }
        p[OUT_H] = 1; p[OUT_W] = p[IN_H] * p[IN_W] * (p[IN_C] / p[OUT_C]);
        return 0;
    case APPEND_LAYER:
    {
        if (L->parent_idx[PARENT_1] < 0) { ERROR_PRTF ("layer %u: append without from=\n", L->layer_idx); return -1; }
        if (p[STRIDE] == 0) p[STRIDE] = 1;
        const aspen_layer_t *Q = &dnn->layers[L->parent_idx[PARENT_1]];
        p[OUT_C] = p[IN_C] + Q->params[OUT_C]; p[OUT_H] = p[IN_H] * p[STRIDE]; p[OUT_W] = p[IN_W] * p[STRIDE];
        if (Q->params[OUT_H] != p[OUT_H] || Q->params[OUT_W] != p[OUT_W])
        { ERROR_PRTF ("layer %u: append: the second parent is %ux%u, the upsampled first parent %ux%u\n", L->layer_idx, Q->params[OUT_H], Q->params[OUT_W], p[OUT_H], p[OUT_W]); return -1; }
        return 0;
    }
    case K_ATTENTION_LAYER:
        if (L->parent_idx[PARENT_1] < 0 || p[NUM_HEAD] == 0 || p[NUM_HIDDEN] == 0) { ERROR_PRTF ("layer %u: attention_k needs from=, n_head= and n_embd=\n", L->layer_idx); return -1; }
        p[MAT_K] = p[NUM_HIDDEN] / p[NUM_HEAD];
        return 0;
    default:
        ERROR_PRTF ("ERROR: Unsupported layer type %d at layer %u\n", (int)L->type, L->layer_idx);
        return -1;
    }
}

/* Checks a layer whose parents and parameters came from a file instead of a cfg section: parent indices
   point at earlier layers, no dimension is absurd, and the geometry the file states is the one the layer's
   parents and window parameters imply (the same derivation a cfg section goes through).  Layers
   0 .. layer_idx-1 of the model must already have passed. */
int aspen_layer_validate (aspen_dnn_t *dnn, aspen_layer_t *L)
{
    const unsigned int i = L->layer_idx;
    if (L->type == INPUT_LAYER ? i != 0 : (i == 0 || L->parent_idx[PARENT_0] < 0 || L->parent_idx[PARENT_0] >= (int)i))
    { ERROR_PRTF ("layer %u: bad first parent %d\n", i, L->parent_idx[PARENT_0]); return -1; }
    if (L->parent_idx[PARENT_1] >= (int)i || L->parent_idx[PARENT_1] < -1)
    { ERROR_PRTF ("layer %u: bad second parent %d\n", i, L->parent_idx[PARENT_1]); return -1; }
    for (int k = 0; k < NUM_PARAM_ELEMENTS; k++)
        if (L->params[k] > (1u << 24)) { ERROR_PRTF ("layer %u: parameter %d = %u is out of range\n", i, k, L->params[k]); return -1; }
    unsigned int filed[NUM_PARAM_ELEMENTS];
    memcpy (filed, L->params, sizeof (filed));
    if (set_inout (dnn, L)) return -1;
    static const int geometry[] = { OUT_H, OUT_W, OUT_C, IN_H, IN_W, IN_C, STRIDE };
    /* layer kinds whose geometry follows from their parents' (image layers; the transformer kinds carry their
       matrix extents as parameters of their own) */
    const int derived = L->type == CONV_LAYER || L->type == MAXPOOL_LAYER || L->type == AVGPOOL_LAYER || L->type == FC_LAYER
        || L->type == YOLO_LAYER || L->type == APPEND_LAYER
        || ((L->type == INPUT_LAYER || L->type == RESIDUAL_LAYER || L->type == SOFTMAX_LAYER) && filed[MAT_M] == 0);
    for (unsigned int k = 0; derived && k < sizeof (geometry) / sizeof (geometry[0]); k++)
    {
        const int g = geometry[k];
        if (g == STRIDE && filed[STRIDE] == 0) continue;                       /* 0 means 1, as in a cfg section */
        if (g == OUT_C && (L->type == CONV_LAYER || L->type == FC_LAYER)) continue;      /* free: the number of filters */
        if (L->type == INPUT_LAYER && g >= IN_W) continue;
        if (filed[g] != L->params[g])
        {
            ERROR_PRTF ("layer %u: the file states parameter %s = %u, the layer's parents and window imply %u\n",
                i, param_type_str[g], filed[g], L->params[g]);
            return -1;
        }
    }
    if ((L->type == MATMUL_LAYER || L->type == K_ATTENTION_LAYER) && filed[MAT_K] != L->params[MAT_K])
    { ERROR_PRTF ("layer %u: the file states K = %u, the layer's parent implies %u\n", i, filed[MAT_K], L->params[MAT_K]); return -1; }
    /* what was compared is equal; everything else stays as the file has it */
    const unsigned int stride = L->params[STRIDE];
    memcpy (L->params, filed, sizeof (filed));
    if (derived && filed[STRIDE] == 0) L->params[STRIDE] = stride;
    return 0;
}

aspen_dnn_t *aspen_parse_cfg (const char *path)
{
    const char *ext = strrchr (path, '.');
    if (ext == NULL || strcmp (ext, ".cfg") != 0) { ERROR_PRTF ("Input file type not supported: %s\n", path); return NULL; }
    int n = 0;
    section_t *secs = read_sections (path, &n);
    if (secs == NULL) return NULL;
    if (n == 0 || section_type (secs[0].name) != INPUT_LAYER)
    {
        ERROR_PRTF ("First section must be [net] or [network]\n");
        free (secs);
        return NULL;
    }
    aspen_dnn_t *dnn = calloc (1, sizeof (aspen_dnn_t));
    if (dnn == NULL) { ERROR_PRTF ("Out of host memory reading %s\n", path); free (secs); return NULL; }
    strncpy (dnn->name, path, MAX_STRING_LEN - 1);
    dnn->element_size = sizeof (float);
    dnn->num_layers = n;
    dnn->layers = calloc (n, sizeof (aspen_layer_t));
    if (dnn->layers == NULL) { ERROR_PRTF ("Out of host memory reading %s\n", path); free (dnn); free (secs); return NULL; }
    int bad = 0;
    for (int i = 0; i < n && !bad; i++)
    {
        const section_t *s = &secs[i];
        aspen_layer_t *L = &dnn->layers[i];
        unsigned int *p = L->params;
        L->dnn = dnn; L->layer_idx = i;
        L->type = section_type (s->name);
        p[IN_W] = opt_int (s, "width", 0); p[IN_H] = opt_int (s, "height", 0); p[IN_C] = opt_int (s, "channels", 0);
        p[WEIGHT_W] = p[WEIGHT_H] = opt_int (s, "size", 0);
        p[OUT_C] = opt_int (s, "filters", 0);
        if (p[OUT_C] == 0) p[OUT_C] = opt_int (s, "output", 0);
        p[STRIDE] = opt_int (s, "stride", 0); p[PADDING] = opt_int (s, "pad", 0); p[DILATION] = opt_int (s, "dilation", 0);
        p[MAT_M] = opt_int (s, "M", 0); p[MAT_N] = opt_int (s, "N", 0); p[MAT_K] = opt_int (s, "K", 0);
        p[NUM_HIDDEN] = opt_int (s, "n_embd", 0); p[NUM_HEAD] = opt_int (s, "n_head", 0); p[MASKED] = opt_int (s, "masked", 0);
        L->activation = activation_type (opt_str (s, "activation"));
        for (int k = 0; k < NUM_PARENT_ELEMENTS; k++) L->parent_idx[k] = -1;
        if (L->type != INPUT_LAYER)
        {
            int rel = opt_int (s, "parent", 0);
            L->parent_idx[PARENT_0] = rel ? i + rel : i - 1;
            int from = opt_int (s, "from", 0);
            if (from) L->parent_idx[PARENT_1] = i + from;
            for (int k = PARENT_0; k <= PARENT_1; k++)
                if (L->parent_idx[k] >= i || (k == PARENT_0 && L->parent_idx[k] < 0) || L->parent_idx[k] < -1)
                { ERROR_PRTF ("layer %d: parent offset points outside the preceding layers\n", i); bad = 1; }
        }
        else if (i != 0) { ERROR_PRTF ("layer %d: only the first section may be [net]\n", i); bad = 1; }
        if (L->type == YOLO_LAYER && parse_yolo (s, L)) bad = 1;
        if (!bad && set_inout (dnn, L)) bad = 1;
    }
    free (secs);
    if (bad)
    {
        free (dnn->layers);
        free (dnn);
        return NULL;
    }
    return dnn;
}
