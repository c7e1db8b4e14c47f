/*
 * fileio.c -- the reference's two container formats.
 *
 *   .aspen  a whole model: layers (type, activation, parents, parameters) and their tensors
 *           (reference src/apu_file_io.c:434-809: apu_save_dnn_to_file, apu_parse_dnn_from_file)
 *   .nasm   a tile graph: header (batch, tiles per layer, FLOPs, sequence length) and, per tile, its
 *           parents and children (reference src/apu_file_io.c:811-1093)
 *
 * Both are written exactly in the reference's layout, so files travel in both directions.  Tensors
 * in a .aspen file are stored as the reference keeps them in memory after apu_create_dnn: weights
 * interleaved 8 rows at a time ([M/8][K][8], reference src/apu.c:14-40) with their dimension order
 * spelled out; the reader decodes ANY dimension order the file declares, so files saved by the
 * reference load as well as files saved here.  A .nasm file pins the tile grid of the build that
 * wrote it: a file written by this library is cross-checked tile by tile against the graph the
 * header regenerates; a file written by the reference (CPU tile grid) contributes its header only.
 */
#include "internal.h"

#define VEC_M 8     /* rows interleaved in the reference's packed weights (_VEC_SIZE_M, reference include/aspen.h:33) */

static char *next_line (FILE *fp, char *buf, const char *tag)
{
    if (fgets (buf, MAX_STRING_LEN, fp) == NULL) { ERROR_PRTF ("ASPEN file parse error: unexpected EOF, expected \"%s\".\n", tag); return NULL; }
    buf[strcspn (buf, "\n")] = 0;
    char *p = buf;
    while (*p == ' ' || *p == '\t') p++;
    if (strncmp (p, tag, strlen (tag)) != 0) { ERROR_PRTF ("Wrong ASPEN file format: expected \"%s\", got \"%s\"\n", tag, p); return NULL; }
    return p + strlen (tag);
}

static int next_pair (FILE *fp, char *buf, int *a, int *b)
{
    if (fgets (buf, MAX_STRING_LEN, fp) == NULL) return -1;
    return sscanf (buf, " %d %d", a, b) == 2 ? 0 : -1;
}

/* ---------------------------------------------------------------------------------------------- */
/* .aspen                                                                                          */
/* ---------------------------------------------------------------------------------------------- */
static void write_tensor (FILE *fp, int slot, const LAYER_PARAMS *order, int num_dims, const unsigned int *dims, const float *data, size_t n)
{
    fprintf (fp, "\t\t%d 1\n", slot);
    fprintf (fp, "\t\tNUM_DIMS:%d\n", num_dims);
    fprintf (fp, "\t\tDATA_DIM_ORDER:\n");
    for (int k = 0; k < MAX_TENSOR_DIMS; k++) fprintf (fp, "\t\t\t%d %d\n", k, k < num_dims ? (int)order[k] : 0);
    fprintf (fp, "\t\tDATA_DIM_ORDER_END\n");
    fprintf (fp, "\t\tTENSOR_DIMS:\n");
    for (int k = 0; k < NUM_PARAM_ELEMENTS; k++) fprintf (fp, "\t\t\t%d %u\n", k, dims[k]);
    fprintf (fp, "\t\tTENSOR_DIMS_END\n");
    fprintf (fp, "\t\tTENSOR_DATA:\n");
    fwrite (data, sizeof (float), n, fp);
    fprintf (fp, "\t\tTENSOR_DATA_END\n");
}

void apu_save_dnn_to_file (aspen_dnn_t *dnn, char *filename)
{
    if (dnn == NULL || filename == NULL) { ERROR_PRTF ("apu_save_dnn_to_file: NULL argument.\n"); return; }
    FILE *fp = fopen (filename, "wb");
    if (fp == NULL) { ERROR_PRTF ("Error: apu_save_dnn_to_file Failed to open file %s for writing\n", filename); return; }
    fprintf (fp, "ASPEN_DNN\n");
    fprintf (fp, "ASPEN_BUILD:aspen_amd gfx950\n");
    fprintf (fp, "DNN_NAME:%s\n", dnn->name);
    fprintf (fp, "DNN_ELEMENT_SIZE:%u\n", dnn->element_size);
    fprintf (fp, "NUM_LAYERS:%u\n", dnn->num_layers);
    for (unsigned int i = 0; i < dnn->num_layers; i++)
    {
        const aspen_layer_t *L = &dnn->layers[i];
        const unsigned int *p = L->params;
        fprintf (fp, "\tLAYER_IDX:%u\n\tLAYER_TYPE:%d\n\tLAYER_ACTIVATION:%d\n", L->layer_idx, L->type, L->activation);
        fprintf (fp, "\tLAYER_PARENTS:\n");
        for (int j = 0; j < NUM_PARENT_ELEMENTS; j++) fprintf (fp, "\t\t%d %d\n", j, L->parent_idx[j]);
        fprintf (fp, "\tLAYER_PARENTS_END\n\tLAYER_PARAMS:\n");
        for (int j = 0; j < NUM_PARAM_ELEMENTS; j++) fprintf (fp, "\t\t%d %u\n", j, p[j]);
        fprintf (fp, "\tLAYER_PARAMS_END\n\tLAYER_TENSORS:\n");
        const int weighted = L->weight.data != NULL && (L->type == CONV_LAYER || L->type == FC_LAYER || L->type == MATMUL_LAYER || L->type == LAYERNORM_LAYER);
        for (int j = 0; j < NUM_TENSORS; j++)
        {
            unsigned int dims[NUM_PARAM_ELEMENTS] = {0};
            if (weighted && j == WEIGHT_TENSOR && L->type != LAYERNORM_LAYER)
            {
                /* [M/8][K][8], K in the order the dimension list spells out */
                const unsigned int M = L->gemm_m, K = L->gemm_k, G = (M + VEC_M - 1) / VEC_M;
                float *packed = calloc ((size_t)G * K * VEC_M, sizeof (float));
                if (packed == NULL)
                {
                    ERROR_PRTF ("Error: apu_save_dnn_to_file: out of host memory; %s is incomplete.\n", filename);
                    fclose (fp);
                    return;
                }
                for (unsigned int m = 0; m < M; m++)
                    for (unsigned int k = 0; k < K; k++)
                        packed[((size_t)(m / VEC_M) * K + k) * VEC_M + m % VEC_M] = L->weight.data[(size_t)m * K + k];
                if (L->type == CONV_LAYER)
                {
                    const LAYER_PARAMS order[] = {OUT_C, WEIGHT_H, WEIGHT_W, IN_C, SUB_C};
                    dims[OUT_C] = G; dims[WEIGHT_H] = p[WEIGHT_H]; dims[WEIGHT_W] = p[WEIGHT_W]; dims[IN_C] = p[IN_C]; dims[SUB_C] = VEC_M;
                    write_tensor (fp, j, order, 5, dims, packed, (size_t)G * K * VEC_M);
                }
                else if (L->type == FC_LAYER)
                {
                    const LAYER_PARAMS order[] = {OUT_C, IN_H, IN_W, IN_C, SUB_C};
                    dims[OUT_C] = G; dims[IN_H] = p[IN_H]; dims[IN_W] = p[IN_W]; dims[IN_C] = p[IN_C]; dims[SUB_C] = VEC_M;
                    write_tensor (fp, j, order, 5, dims, packed, (size_t)G * K * VEC_M);
                }
                else
                {
                    const LAYER_PARAMS order[] = {MAT_M, MAT_K, SUB_M};
                    dims[MAT_M] = G; dims[MAT_K] = K; dims[SUB_M] = VEC_M;
                    write_tensor (fp, j, order, 3, dims, packed, (size_t)G * K * VEC_M);
                }
                free (packed);
            }
            else if (weighted && (j == BIAS_TENSOR || (j == WEIGHT_TENSOR && L->type == LAYERNORM_LAYER)))
            {
                const LAYER_PARAMS rows = (L->type == CONV_LAYER || L->type == FC_LAYER) ? OUT_C : MAT_M;
                dims[rows] = L->gemm_m;
                write_tensor (fp, j, &rows, 1, dims, j == BIAS_TENSOR ? L->bias.data : L->weight.data, L->gemm_m);
            }
            else if (L->type == YOLO_LAYER && j == ANCHOR_TENSOR)
            {
                const LAYER_PARAMS rows = OUT_C;        /* as the reference creates it: one dimension of 6 (src/darknet_parser.c:536-541) */
                dims[OUT_C] = 6;
                write_tensor (fp, j, &rows, 1, dims, L->anchors, 6);
            }
            else
                fprintf (fp, "\t\t%d -1\n", j);
        }
        fprintf (fp, "\tLAYER_TENSORS_END\n");
    }
    fprintf (fp, "ASPEN_DNN_END\n");
    fclose (fp);
}

/* position of element `idx` of a tensor with the given dimension order (slowest first) and sizes */
static void decode_pos (size_t idx, const int *order, int num_dims, const unsigned int *dims, unsigned int *pos)
{
    for (int d = num_dims - 1; d >= 0; d--)
    {
        const unsigned int n = dims[order[d]];
        pos[order[d]] = (unsigned int)(idx % n);
        idx /= n;
    }
}

static int place_tensor (aspen_layer_t *L, int slot, const int *order, int num_dims, const unsigned int *dims, const float *data, size_t n)
{
    const unsigned int *p = L->params;
    const int contraction = L->type == CONV_LAYER || L->type == FC_LAYER || L->type == MATMUL_LAYER;
    if (slot == WEIGHT_TENSOR && contraction)
    {
        for (size_t e = 0; e < n; e++)
        {
            unsigned int pos[NUM_PARAM_ELEMENTS] = {0};
            decode_pos (e, order, num_dims, dims, pos);
            size_t m, k;
            if (L->type == MATMUL_LAYER)
            {
                m = dims[SUB_M] > 0 ? (size_t)pos[MAT_M] * dims[SUB_M] + pos[SUB_M] : pos[MAT_M];
                k = pos[MAT_K];
            }
            else
            {
                m = dims[SUB_C] > 0 ? (size_t)pos[OUT_C] * dims[SUB_C] + pos[SUB_C] : pos[OUT_C];
                k = L->type == CONV_LAYER ? ((size_t)pos[WEIGHT_H] * p[WEIGHT_W] + pos[WEIGHT_W]) * p[IN_C] + pos[IN_C]
                                          : ((size_t)pos[IN_H] * p[IN_W] + pos[IN_W]) * p[IN_C] + pos[IN_C];
            }
            if (m >= L->gemm_m) continue;                 /* padding rows of the last interleaved group */
            if (k >= L->gemm_k) return -1;
            L->weight.data[m * L->gemm_k + k] = data[e];
        }
        return 0;
    }
    if (slot == BIAS_TENSOR || (slot == WEIGHT_TENSOR && L->type == LAYERNORM_LAYER))
    {
        aspen_tensor_t *t = slot == BIAS_TENSOR ? &L->bias : &L->weight;
        if (t->data == NULL || n < L->gemm_m) return -1;
        memcpy (t->data, data, L->gemm_m * sizeof (float));
        return 0;
    }
    if (slot == ANCHOR_TENSOR && L->type == YOLO_LAYER)
    {
        if (n < 6) return -1;
        memcpy (L->anchors, data, 6 * sizeof (float));
        return 0;
    }
    return 0;    /* tensors this build has no use for (anchors, BN statistics already folded) are skipped */
}

int aspen_create_layer_tensors (aspen_layer_t *L);      /* dnn.c */

aspen_dnn_t *apu_load_dnn_from_file (char *filename)
{
    if (filename == NULL) { ERROR_PRTF ("apu_load_dnn_from_file: filename is NULL.\n"); return NULL; }
    FILE *fp = fopen (filename, "rb");
    if (fp == NULL) { ERROR_PRTF ("ASPEN DNN file %s not found.\n", filename); return NULL; }
    char line[MAX_STRING_LEN];
    char *ptr;
    aspen_dnn_t *dnn = NULL;
    float *data = NULL;
    if (next_line (fp, line, "ASPEN_DNN") == NULL || next_line (fp, line, "ASPEN_BUILD:") == NULL) goto fail;
    if ((ptr = next_line (fp, line, "DNN_NAME:")) == NULL) goto fail;
    dnn = calloc (1, sizeof (aspen_dnn_t));
    if (dnn == NULL) goto fail;
    strncpy (dnn->name, ptr, MAX_STRING_LEN - 1);
    if ((ptr = next_line (fp, line, "DNN_ELEMENT_SIZE:")) == NULL) goto fail;
    dnn->element_size = (unsigned int)atoi (ptr);
    if (dnn->element_size != sizeof (float)) { ERROR_PRTF ("ASPEN DNN file %s: element size %u is not supported.\n", filename, dnn->element_size); goto fail; }
    if ((ptr = next_line (fp, line, "NUM_LAYERS:")) == NULL) goto fail;
    dnn->num_layers = (unsigned int)atoi (ptr);
    if (dnn->num_layers == 0 || dnn->num_layers > 65535) goto fail;
    dnn->layers = calloc (dnn->num_layers, sizeof (aspen_layer_t));
    if (dnn->layers == NULL) { dnn->num_layers = 0; goto fail; }
    for (unsigned int i = 0; i < dnn->num_layers; i++)
    {
        aspen_layer_t *L = &dnn->layers[i];
        L->dnn = dnn;
        if ((ptr = next_line (fp, line, "LAYER_IDX:")) == NULL) goto fail;
        L->layer_idx = (unsigned int)atoi (ptr);
        if ((ptr = next_line (fp, line, "LAYER_TYPE:")) == NULL) goto fail;
        L->type = (LAYER_TYPE)atoi (ptr);
        if ((int)L->type < 0 || (int)L->type >= NUM_LAYER_ELEMENTS) { ERROR_PRTF ("ASPEN DNN file %s: layer %u has unknown type %d.\n", filename, i, (int)L->type); goto fail; }
        if ((ptr = next_line (fp, line, "LAYER_ACTIVATION:")) == NULL) goto fail;
        L->activation = (LAYER_ACT)atoi (ptr);
        if ((int)L->activation < 0 || (int)L->activation >= NUM_ACTIVATIONS) { ERROR_PRTF ("ASPEN DNN file %s: layer %u has unknown activation %d.\n", filename, i, (int)L->activation); goto fail; }
        if (next_line (fp, line, "LAYER_PARENTS:") == NULL) goto fail;
        for (int j = 0; j < NUM_PARENT_ELEMENTS; j++)
        {
            int a, b;
            if (next_pair (fp, line, &a, &b) || a < 0 || a >= NUM_PARENT_ELEMENTS || b >= (int)i) goto fail;
            L->parent_idx[a] = b;
        }
        if (next_line (fp, line, "LAYER_PARENTS_END") == NULL || next_line (fp, line, "LAYER_PARAMS:") == NULL) goto fail;
        for (int j = 0; j < NUM_PARAM_ELEMENTS; j++)
        {
            int a, b;
            if (next_pair (fp, line, &a, &b) || a < 0 || a >= NUM_PARAM_ELEMENTS) goto fail;
            L->params[a] = (unsigned int)b;
        }
        if (next_line (fp, line, "LAYER_PARAMS_END") == NULL || next_line (fp, line, "LAYER_TENSORS:") == NULL) goto fail;
        if (L->layer_idx != i) { ERROR_PRTF ("ASPEN DNN file %s: layer %u carries index %u.\n", filename, i, L->layer_idx); goto fail; }
        /* the tensors are sized from these parameters and the kernels index with them */
        if (aspen_layer_validate (dnn, L)) { ERROR_PRTF ("ASPEN DNN file %s: layer %u has inconsistent parameters.\n", filename, i); goto fail; }
        if (aspen_create_layer_tensors (L)) goto fail;
        for (int j = 0; j < NUM_TENSORS; j++)
        {
            int slot, present;
            if (next_pair (fp, line, &slot, &present)) goto fail;
            if (present == -1) continue;
            int order[MAX_TENSOR_DIMS] = {0}, num_dims;
            unsigned int dims[NUM_PARAM_ELEMENTS] = {0};
            if ((ptr = next_line (fp, line, "NUM_DIMS:")) == NULL) goto fail;
            num_dims = atoi (ptr);
            if (num_dims < 1 || num_dims > MAX_TENSOR_DIMS || next_line (fp, line, "DATA_DIM_ORDER:") == NULL) goto fail;
            for (int k = 0; k < MAX_TENSOR_DIMS; k++)
            {
                int a, b;
                if (next_pair (fp, line, &a, &b) || a < 0 || a >= MAX_TENSOR_DIMS || b < 0 || b >= NUM_PARAM_ELEMENTS) goto fail;
                order[a] = b;
            }
            if (next_line (fp, line, "DATA_DIM_ORDER_END") == NULL || next_line (fp, line, "TENSOR_DIMS:") == NULL) goto fail;
            for (int k = 0; k < NUM_PARAM_ELEMENTS; k++)
            {
                int a, b;
                if (next_pair (fp, line, &a, &b) || a < 0 || a >= NUM_PARAM_ELEMENTS || b < 0) goto fail;
                dims[a] = (unsigned int)b;
            }
            if (next_line (fp, line, "TENSOR_DIMS_END") == NULL || next_line (fp, line, "TENSOR_DATA:") == NULL) goto fail;
            size_t n = 1;
            for (int k = 0; k < num_dims; k++) n *= dims[order[k]];
            if (n == 0 || n > ((size_t)1 << 33)) goto fail;
            data = malloc (n * sizeof (float));
            if (data == NULL || fread (data, sizeof (float), n, fp) != n) { ERROR_PRTF ("ASPEN DNN file %s parse error: Failed to read tensor data.\n", filename); goto fail; }
            if (place_tensor (L, slot, order, num_dims, dims, data, n))
            { ERROR_PRTF ("ASPEN DNN file %s: tensor %d of layer %u does not fit the layer.\n", filename, slot, i); goto fail; }
            free (data); data = NULL;
            if (next_line (fp, line, "TENSOR_DATA_END") == NULL) goto fail;
        }
        if (next_line (fp, line, "LAYER_TENSORS_END") == NULL) goto fail;
    }
    if (next_line (fp, line, "ASPEN_DNN_END") == NULL) goto fail;
    fclose (fp);
    return dnn;
fail:
    ERROR_PRTF ("ASPEN DNN file %s could not be loaded.\n", filename);
    free (data);
    fclose (fp);
    if (dnn) { dnn->ref_nasms = 0; apu_destroy_dnn (dnn); }
    return NULL;
}

/* ---------------------------------------------------------------------------------------------- */
/* .nasm                                                                                           */
/* ---------------------------------------------------------------------------------------------- */
/* parents of every tile as CSR, derived from the children lists */
static void parent_lists (const nasm_t *nasm, uint32_t **off_out, uint32_t **idx_out)
{
    const uint32_t n = nasm->num_ninst;
    uint32_t *off = calloc ((size_t)n + 2, sizeof (uint32_t)), *idx = calloc (nasm->num_edges ? nasm->num_edges : 1, sizeof (uint32_t));
    uint32_t *cur = calloc (n ? n : 1, sizeof (uint32_t));
    *off_out = *idx_out = NULL;
    if (off == NULL || idx == NULL || cur == NULL) { free (off); free (idx); free (cur); return; }
    for (uint32_t t = 0; t < n; t++) off[t + 1] = off[t] + nasm->num_parents[t];
    for (uint32_t t = 0; t < n; t++)                       /* parents in increasing order, as tiles are visited in order */
        for (uint32_t c = nasm->child_off[t]; c < nasm->child_off[t + 1]; c++)
        {
            const uint32_t child = nasm->child_idx[c];
            idx[off[child] + cur[child]++] = t;
        }
    free (cur);
    *off_out = off; *idx_out = idx;
}

void apu_save_nasm_to_file (nasm_t *nasm, char *filename)
{
    if (nasm == NULL) { ERROR_PRTF ("ASPEN NASM to save is null.\n"); return; }
    if (filename == NULL) { ERROR_PRTF ("ASPEN NASM file name not specified.\n"); return; }
    FILE *fp = fopen (filename, "wb");
    if (fp == NULL) { ERROR_PRTF ("Error: apu_save_nasm_to_file Failed to open file %s for writing\n", filename); return; }
    uint32_t *poff, *pidx;
    parent_lists (nasm, &poff, &pidx);
    if (poff == NULL) { ERROR_PRTF ("Error: apu_save_nasm_to_file: out of host memory.\n"); fclose (fp); return; }
    fprintf (fp, "ASPEN_NASM\n");
    fprintf (fp, "DNN_NAME:%s\n", nasm->dnn->name);
    fprintf (fp, "NUM_BATCH:%u\n", nasm->batch_size);
    fprintf (fp, "MIN_NINST_PER_LDATA:%u\n", nasm->min_ninst_per_ldata);
    fprintf (fp, "TOTAL_FLOPS:%llu\n", (unsigned long long)nasm->total_flops);
    fprintf (fp, "FLOP_PER_NINST:0\n");                  /* the reference's CPU tile-size target; tiles here are fixed MFMA shapes */
    fprintf (fp, "SEQ_LEN:%u\n", nasm->tr_seq_len);
    fprintf (fp, "NASM_NINSTS:\n");
    for (uint32_t t = 0; t < nasm->num_ninst; t++)
    {
        const uint32_t nc = nasm->child_off[t + 1] - nasm->child_off[t];
        fprintf (fp, "\tNINST_IDX:%u\n\tNUM_CHILD_NINSTS:%u\n\tNUM_PARENT_NINSTS:%u\n\tPARENT_NINSTS:\n", t, nc, nasm->num_parents[t]);
        for (uint32_t k = 0; k < nasm->num_parents[t]; k++) fprintf (fp, "\t\t%u %u\n", k, pidx[poff[t] + k]);
        fprintf (fp, "\tPARENT_NINSTS_END\n\tNUM_CHILD_NINSTS:%u\n\tCHILD_NINST_IDXES:\n", nc);
        for (uint32_t k = 0; k < nc; k++) fprintf (fp, "\t\t%u %u\n", k, nasm->child_idx[nasm->child_off[t] + k]);
        fprintf (fp, "\tCHILD_NINST_IDXES_END\n\tNUM_INPUT_POS:0\n");
    }
    fprintf (fp, "NASM_NINSTS_END\nASPEN_NASM_END\n");
    fclose (fp);
    free (poff); free (pidx);
}

nasm_t *apu_load_nasm_from_file (char *filename, aspen_dnn_t *dnn)
{
    if (dnn == NULL) { ERROR_PRTF ("ASPEN DNN NASM load error: dnn is null.\n"); return NULL; }
    if (filename == NULL) { ERROR_PRTF ("ASPEN DNN NASM load error: filename is null.\n"); return NULL; }
    FILE *fp = fopen (filename, "rb");
    if (fp == NULL) { ERROR_PRTF ("ASPEN DNN NASM load error: file %s not found.\n", filename); return NULL; }
    char line[MAX_STRING_LEN];
    char *ptr;
    unsigned int batch, min_ninst, seq;
    unsigned long long flops;
    nasm_t *nasm = NULL;
    uint32_t *poff = NULL, *pidx = NULL;
    if (next_line (fp, line, "ASPEN_NASM") == NULL) { ERROR_PRTF ("ASPEN DNN file %s parse error: Not an ASPEN NASM file.\n", filename); goto fail; }
    if (next_line (fp, line, "DNN_NAME:") == NULL) goto fail;            /* a differing name is tolerated, as in the reference */
    if ((ptr = next_line (fp, line, "NUM_BATCH:")) == NULL) goto fail;
    batch = (unsigned int)atoi (ptr);
    if ((ptr = next_line (fp, line, "MIN_NINST_PER_LDATA:")) == NULL) goto fail;
    min_ninst = (unsigned int)atoi (ptr);
    if ((ptr = next_line (fp, line, "TOTAL_FLOPS:")) == NULL) goto fail;
    flops = strtoull (ptr, NULL, 10);
    if (next_line (fp, line, "FLOP_PER_NINST:") == NULL) goto fail;
    if ((ptr = next_line (fp, line, "SEQ_LEN:")) == NULL) goto fail;
    seq = (unsigned int)atoi (ptr);
    if (next_line (fp, line, "NASM_NINSTS:") == NULL) goto fail;
    nasm = seq ? apu_create_transformer_nasm (dnn, min_ninst ? min_ninst : 1, batch, seq) : apu_create_nasm (dnn, min_ninst ? min_ninst : 1, batch);
    if (nasm == NULL) goto fail;
    if (flops != 0 && flops != nasm->total_flops)
    {
        ERROR_PRTF ("ASPEN NASM file %s: TOTAL_FLOPS %llu does not match the model (%llu): wrong dnn or batch.\n",
            filename, flops, (unsigned long long)nasm->total_flops);
        goto fail;
    }
    /* the tile list: cross-checked when it is this build's grid, skipped when it is another build's */
    parent_lists (nasm, &poff, &pidx);
    if (poff == NULL) goto fail;
    uint32_t count = 0;
    int own_grid = 1, mismatch = 0;
    for (;;)
    {
        if (fgets (line, MAX_STRING_LEN, fp) == NULL) { ERROR_PRTF ("ASPEN NASM file %s parse error: unexpected EOF.\n", filename); goto fail; }
        char *p = line;
        while (*p == ' ' || *p == '\t') p++;
        if (strncmp (p, "NASM_NINSTS_END", 15) == 0) break;
        if (strncmp (p, "NINST_IDX:", 10) != 0) { ERROR_PRTF ("ASPEN NASM file %s parse error: expected NINST_IDX, got \"%s\"\n", filename, p); goto fail; }
        const uint32_t idx = (uint32_t)atoi (p + 10);
        if (idx != count) { ERROR_PRTF ("ASPEN NASM file %s: NINST_IDX %u out of order.\n", filename, idx); goto fail; }
        unsigned int nc, np;
        if ((ptr = next_line (fp, line, "NUM_CHILD_NINSTS:")) == NULL) goto fail;
        nc = (unsigned int)atoi (ptr);
        if ((ptr = next_line (fp, line, "NUM_PARENT_NINSTS:")) == NULL) goto fail;
        np = (unsigned int)atoi (ptr);
        if (next_line (fp, line, "PARENT_NINSTS:") == NULL) goto fail;
        const int check = own_grid && idx < nasm->num_ninst;
        if (check && (np != nasm->num_parents[idx] || nc != nasm->child_off[idx + 1] - nasm->child_off[idx])) own_grid = 0;
        for (unsigned int k = 0; k < np; k++)
        {
            int a, b;
            if (next_pair (fp, line, &a, &b)) goto fail;
            if (check && own_grid && (uint32_t)b != pidx[poff[idx] + k]) mismatch = 1;
        }
        if (next_line (fp, line, "PARENT_NINSTS_END") == NULL || next_line (fp, line, "NUM_CHILD_NINSTS:") == NULL
            || next_line (fp, line, "CHILD_NINST_IDXES:") == NULL) goto fail;
        for (unsigned int k = 0; k < nc; k++)
        {
            int a, b;
            if (next_pair (fp, line, &a, &b)) goto fail;
            if (check && own_grid && (uint32_t)b != nasm->child_idx[nasm->child_off[idx] + k]) mismatch = 1;
        }
        if (next_line (fp, line, "CHILD_NINST_IDXES_END") == NULL || next_line (fp, line, "NUM_INPUT_POS:") == NULL) goto fail;
        count++;
    }
    if (next_line (fp, line, "ASPEN_NASM_END") == NULL) goto fail;
    if (count != nasm->num_ninst) own_grid = 0;
    if (own_grid && mismatch) { ERROR_PRTF ("ASPEN NASM file %s: tile dependencies differ from the graph its header describes.\n", filename); goto fail; }
    if (!own_grid)
        printf ("ASPEN NASM file %s lists %u tiles of another tile grid; the graph was rebuilt from its header (%u tiles).\n", filename, count, nasm->num_ninst);
    fflush (stdout);
    fclose (fp);
    free (poff); free (pidx);
    return nasm;
fail:
    fclose (fp);
    free (poff); free (pidx);
    if (nasm) apu_destroy_nasm (nasm);
    return NULL;
}
