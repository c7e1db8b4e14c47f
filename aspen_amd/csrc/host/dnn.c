/*
 * dnn.c -- model object: creation, ASPEN_DATA weight files, device-side weight layout.
 *
 * Counterpart of the reference's apu_create_dnn / apu_load_dnn_data_from_file
 * (reference src/apu.c:6-43, src/apu_file_io.c:48-432).  The reference repacks weights into
 * [M/8][K][8] for its 8-row AVX2 micro-kernel; here the device copy is [roundup(M,128)][Kp]
 * row-major with the K axis laid out as (tap, channel padded to 4) so that every 128-bit load of
 * the implicit-GEMM kernel stays inside one tap, zero padded to a multiple of 32.
 */
#include <math.h>
#include "internal.h"

static void alloc_tensor (aspen_tensor_t *t, size_t n)
{
    t->num_elements = n;
    t->data = calloc (n ? n : 1, sizeof (float));
}

/* deterministic stand-in for the reference's rand()-based +-0.3 fill (reference src/apu.c:345-354,
   :419-421): weights a model has before any file is loaded */
static void fill_uniform (aspen_tensor_t *t, uint64_t *state, float range)
{
    for (size_t i = 0; i < t->num_elements; i++)
    {
        *state = *state * 6364136223846793005ull + 1442695040888963407ull;
        t->data[i] = ((float)((*state >> 40) & 0xffffff) / 16777216.0f - 0.5f) * 2.0f * range;
    }
}

static int create_layer_tensors (aspen_layer_t *L, uint64_t *rng)
{
    const unsigned int *p = L->params;
    switch (L->type)
    {
    case CONV_LAYER:    L->gemm_m = p[OUT_C]; L->gemm_k = p[WEIGHT_H] * p[WEIGHT_W] * p[IN_C]; break;
    case FC_LAYER:      L->gemm_m = p[OUT_C]; L->gemm_k = p[IN_H] * p[IN_W] * p[IN_C]; break;
    case MATMUL_LAYER:  L->gemm_m = p[MAT_M]; L->gemm_k = p[MAT_K]; break;
    case LAYERNORM_LAYER: L->gemm_m = p[MAT_M]; L->gemm_k = 1; break;
    default: return 0;
    }
    alloc_tensor (&L->weight, (size_t)L->gemm_m * L->gemm_k);
    alloc_tensor (&L->bias, L->gemm_m);
    if (L->weight.data == NULL || L->bias.data == NULL)
    {
        ERROR_PRTF ("layer %u: out of host memory for %zu weights\n", L->layer_idx, (size_t)L->gemm_m * L->gemm_k);
        free (L->weight.data); free (L->bias.data);
        L->weight.data = L->bias.data = NULL; L->weight.num_elements = L->bias.num_elements = 0;
        return -1;
    }
    fill_uniform (&L->weight, rng, 0.3f);
    fill_uniform (&L->bias, rng, 0.3f);
    return 0;
}

/* tensors of a layer whose parameters are known, zero filled (the .aspen reader fills them) */
int aspen_create_layer_tensors (aspen_layer_t *L)
{
    uint64_t rng = 1;
    if (create_layer_tensors (L, &rng)) return -1;
    if (L->weight.data) memset (L->weight.data, 0, L->weight.num_elements * sizeof (float));
    if (L->bias.data) memset (L->bias.data, 0, L->bias.num_elements * sizeof (float));
    return 0;
}

aspen_dnn_t *apu_create_dnn (char *input_path, char *data_path)
{
    if (input_path == NULL) { ERROR_PRTF ("apu_create_dnn: input_path is NULL\n"); return NULL; }
    aspen_dnn_t *dnn = aspen_parse_cfg (input_path);
    if (dnn == NULL) return NULL;
    uint64_t rng = 0x5851f42d4c957f2dull;
    for (unsigned int i = 0; i < dnn->num_layers; i++)
        if (create_layer_tensors (&dnn->layers[i], &rng)) { apu_destroy_dnn (dnn); return NULL; }
    if (data_path != NULL)
        aspen_load_weight_file (dnn, data_path);   /* a missing or broken file only prints, as in the reference */
    return dnn;
}

/* reference include/apu.h:46 (src/apu_file_io.c:48): loads an ASPEN_DATA weight file into an existing model,
   also one whose graphs have already run: the layers' device copies are dropped, and every ready pool that
   holds a graph of this model rebuilds its device graph before its next run. */
void apu_load_dnn_data_from_file (aspen_dnn_t *dnn, char *input_path)
{
    if (dnn == NULL || input_path == NULL) { ERROR_PRTF ("apu_load_dnn_data_from_file: NULL argument\n"); return; }
    aspen_hip_sync ();                 /* nothing in flight may still read the buffers about to be released */
    aspen_load_weight_file (dnn, input_path);
}

void apu_destroy_dnn (aspen_dnn_t *dnn)
{
    if (dnn == NULL) return;
    if (dnn->ref_nasms != 0)
    {
        ERROR_PRTF ("Cannot destroy dnn %s with %d nasms still referencing it.\n", dnn->name, dnn->ref_nasms);
        return;
    }
    for (unsigned int i = 0; i < dnn->num_layers; i++)
    {
        aspen_layer_t *L = &dnn->layers[i];
        free (L->weight.data); free (L->bias.data);
        aspen_hip_free (L->d_weight); aspen_hip_free (L->d_bias); aspen_hip_free (L->d_ktab);
    }
    free (dnn->layers);
    free (dnn);
}

/* ---------------------------------------------------------------------------------------------- */
/* ASPEN_DATA reader                                                                               */
/* ---------------------------------------------------------------------------------------------- */
static char *expect_line (FILE *fp, char *buf, size_t len, const char *tag, int eof_ok)
{
    if (fgets (buf, (int)len, fp) == NULL)
    {
        if (!eof_ok) ERROR_PRTF ("ASPEN DNN file parse error: Unexpected EOF.\n");
        return NULL;
    }
    buf[strcspn (buf, "\n")] = 0;
    char *p = buf;
    while (*p == ' ' || *p == '\t') p++;
    if (strncmp (p, tag, strlen (tag)) != 0)
    {
        ERROR_PRTF ("Wrong ASPEN DNN file format: expected \"%s\", got \"%s\"\n", tag, p);
        return NULL;
    }
    return p + strlen (tag);
}

/* PyTorch [O][C][H][W] -> GEMM order [O][(h*W + w)*C + c] */
static void ochw_to_ohwc (const float *src, float *dst, unsigned int O, unsigned int C, unsigned int H, unsigned int W)
{
    for (unsigned int o = 0; o < O; o++)
        for (unsigned int c = 0; c < C; c++)
            for (unsigned int h = 0; h < H; h++)
                for (unsigned int w = 0; w < W; w++)
                    dst[((size_t)o * H * W + (size_t)h * W + w) * C + c] = src[(((size_t)o * C + c) * H + h) * W + w];
}

static void invalidate_device (aspen_layer_t *L)
{
    /* device graphs that were built from these buffers must not run again as they are */
    if ((L->d_weight || L->d_bias || L->d_ktab) && L->dnn != NULL) L->dnn->dev_generation++;
    aspen_hip_free (L->d_weight); aspen_hip_free (L->d_bias); aspen_hip_free (L->d_ktab);
    aspen_hip_free (L->d_weight_ln); aspen_hip_free (L->d_bias_ln); aspen_hip_free (L->d_rowsum_ln);
    L->d_weight = NULL; L->d_bias = NULL; L->d_ktab = NULL;
    L->d_weight_ln = NULL; L->d_bias_ln = NULL; L->d_rowsum_ln = NULL;
    /* (a layer norm's parameters are part of what the matmul layers behind it hold folded in) */
    if (L->type == LAYERNORM_LAYER && L->dnn != NULL)
        for (unsigned int i = 0; i < L->dnn->num_layers; i++)
        {
            aspen_layer_t *C = &L->dnn->layers[i];
            if (C->type != MATMUL_LAYER || C->parent_idx[PARENT_0] != (int)L->layer_idx || C->d_weight_ln == NULL) continue;
            aspen_hip_free (C->d_weight_ln); aspen_hip_free (C->d_bias_ln); aspen_hip_free (C->d_rowsum_ln);
            C->d_weight_ln = NULL; C->d_bias_ln = NULL; C->d_rowsum_ln = NULL;
        }
}

int aspen_load_weight_file (aspen_dnn_t *dnn, const char *path)
{
    FILE *fp = fopen (path, "rb");
    if (fp == NULL) { ERROR_PRTF ("ASPEN DNN file %s not found.\n", path); return -1; }
    char line[MAX_STRING_LEN];
    float *bn[3] = {NULL, NULL, NULL};   /* var, mean, weight */
    int rc = -1;
    char *p;
    if (expect_line (fp, line, sizeof (line), "ASPEN_DATA", 0) == NULL) goto done;
    p = expect_line (fp, line, sizeof (line), "LAYER:", 0);
    while (p != NULL)
    {
        const int file_layer = atoi (p);
        aspen_layer_t *L = NULL;
        int weighted = 0;
        for (unsigned int i = 0; i < dnn->num_layers && L == NULL; i++)
        {
            LAYER_TYPE t = dnn->layers[i].type;
            if (t == CONV_LAYER || t == FC_LAYER || t == MATMUL_LAYER || t == LAYERNORM_LAYER)
                if (++weighted == file_layer) L = &dnn->layers[i];
        }
        if (L == NULL) { ERROR_PRTF ("ASPEN DNN file %s parse error: Invalid file LAYER %d.\n", path, file_layer); goto done; }
        if ((p = expect_line (fp, line, sizeof (line), "TENSOR_TYPE:", 0)) == NULL) goto done;
        char kind[32];
        strncpy (kind, p, sizeof (kind) - 1); kind[sizeof (kind) - 1] = 0;
        if ((p = expect_line (fp, line, sizeof (line), "DATA_SIZE:", 0)) == NULL) goto done;
        const size_t bytes = (size_t)atoll (p);
        if (expect_line (fp, line, sizeof (line), "DATA_START:", 0) == NULL) goto done;
        /* the size the tensor must have is known from the layer: checked BEFORE anything is allocated, so a
           file cannot ask for an arbitrary amount of memory */
        size_t expect;
        int skip = 0;
        if (strcmp (kind, "WEIGHT") == 0) expect = L->weight.num_elements * sizeof (float);
        else if (strcmp (kind, "BIAS") == 0) expect = L->bias.num_elements * sizeof (float);
        else if (strcmp (kind, "BN_VAR") == 0 || strcmp (kind, "BN_MEAN") == 0 || strcmp (kind, "BN_WEIGHT") == 0) expect = L->gemm_m * sizeof (float);
        else if (strcmp (kind, "INPUT") == 0 || strcmp (kind, "OUTPUT") == 0) { expect = bytes; skip = 1; }
        else
        {
            ERROR_PRTF ("ASPEN DNN file %s file layer %d parse error: Invalid TENSOR_TYPE %s.\n", path, file_layer, kind);
            goto done;
        }
        if (bytes != expect)
        {
            ERROR_PRTF ("ASPEN DNN file %s parse error: Layer %u %s_TENSOR size mismatch. Tensor: %zu, File: %zu.\n",
                path, L->layer_idx, kind, expect, bytes);
            goto done;
        }
        float *buf = NULL;
        if (skip)
        {
            if (fseek (fp, (long)bytes, SEEK_CUR) != 0) { ERROR_PRTF ("ASPEN DNN file %s parse error: Failed to read data.\n", path); goto done; }
        }
        else
        {
            buf = malloc (bytes ? bytes : 1);
            if (buf == NULL || fread (buf, 1, bytes, fp) != bytes)
            {
                ERROR_PRTF ("ASPEN DNN file %s parse error: Failed to read data.\n", path);
                free (buf);
                goto done;
            }
        }
        if (expect_line (fp, line, sizeof (line), "DATA_END", 0) == NULL) { free (buf); goto done; }
        const unsigned int *q = L->params;
        if (strcmp (kind, "WEIGHT") == 0)
        {
            if (bytes != L->weight.num_elements * sizeof (float))
            {
                ERROR_PRTF ("ASPEN DNN file %s parse error: Layer %u WEIGHT_TENSOR size mismatch. Tensor: %zu, File: %zu.\n",
                    path, L->layer_idx, L->weight.num_elements * sizeof (float), bytes);
                free (buf);
                goto done;
            }
            if (L->type == CONV_LAYER) ochw_to_ohwc (buf, L->weight.data, q[OUT_C], q[IN_C], q[WEIGHT_H], q[WEIGHT_W]);
            else if (L->type == FC_LAYER) ochw_to_ohwc (buf, L->weight.data, q[OUT_C], q[IN_C], q[IN_H], q[IN_W]);
            else memcpy (L->weight.data, buf, bytes);
            invalidate_device (L);
            free (buf);
        }
        else if (strcmp (kind, "BIAS") == 0)
        {
            if (bytes != L->bias.num_elements * sizeof (float))
            {
                ERROR_PRTF ("ASPEN DNN file %s parse error: Layer %u BIAS_TENSOR size mismatch: Tensor: %zu, File: %zu.\n",
                    path, L->layer_idx, L->bias.num_elements * sizeof (float), bytes);
                free (buf);
                goto done;
            }
            memcpy (L->bias.data, buf, bytes);
            invalidate_device (L);
            free (buf);
        }
        else if (strcmp (kind, "BN_VAR") == 0 || strcmp (kind, "BN_MEAN") == 0 || strcmp (kind, "BN_WEIGHT") == 0)
        {
            const int slot = kind[3] == 'V' ? 0 : kind[3] == 'M' ? 1 : 2;
            if (bn[slot] != NULL || bytes != L->gemm_m * sizeof (float))
            {
                ERROR_PRTF ("ASPEN DNN file %s parse error: Duplicate or mis-sized %s.\n", path, kind);
                free (buf);
                goto done;
            }
            bn[slot] = buf;
        }
        else if (strcmp (kind, "INPUT") == 0 || strcmp (kind, "OUTPUT") == 0)
            free (buf);
        else
        {
            ERROR_PRTF ("ASPEN DNN file %s file layer %d parse error: Invalid TENSOR_TYPE %s.\n", path, file_layer, kind);
            free (buf);
            goto done;
        }
        if (bn[0] && bn[1] && bn[2])
        {
            /* fold inference batch norm into weight and bias, eps 1e-5 (reference src/util.c:259-276) */
            const double eps = 1e-5;
            for (unsigned int o = 0; o < L->gemm_m; o++)
            {
                const float s = bn[2][o] / sqrtf (bn[0][o] + eps);
                for (unsigned int k = 0; k < L->gemm_k; k++) L->weight.data[(size_t)o * L->gemm_k + k] *= s;
                L->bias.data[o] = L->bias.data[o] - bn[2][o] * bn[1][o] / sqrtf (bn[0][o] + eps);
            }
            for (int i = 0; i < 3; i++) { free (bn[i]); bn[i] = NULL; }
            invalidate_device (L);
        }
        if (expect_line (fp, line, sizeof (line), "LAYER_END", 0) == NULL) goto done;
        p = expect_line (fp, line, sizeof (line), "LAYER:", 1);
    }
    rc = 0;
done:
    for (int i = 0; i < 3; i++) free (bn[i]);
    fclose (fp);
    return rc;
}

/* ---------------------------------------------------------------------------------------------- */
/* device layout                                                                                    */
/* ---------------------------------------------------------------------------------------------- */
static unsigned int round_up (unsigned int v, unsigned int to) { return (v + to - 1) / to * to; }

/* A convolution over three input channels (a network's first layer on RGB images) keeps its K axis dense on the
   device: K = taps * 3 instead of taps * 4, see ASPEN_HIP_OPERAND_DENSE3.  (The stem of ResNet-50: 160 instead of 224.) */
int aspen_layer_dense3 (const aspen_layer_t *L)
{
    /* read once: the K layout, the table layout and the operand kind of a layer all follow from this answer and must agree */
    static int disabled = -1;
    if (disabled < 0) disabled = getenv ("ASPEN_GPU_NO_DENSE3") != NULL;
    return L->type == CONV_LAYER && L->params[IN_C] == 3 && L->params[WEIGHT_H] * L->params[WEIGHT_W] * 3 <= 508 && L->gemm_m <= 64
        && !disabled;
}

/* A contraction layer whose channel count is not a multiple of the K slice width (32): a slice straddles taps, so
   the kernels resolve its K axis through the k-chunk table, which only the 64 x 64 tile shape can do. */
int aspen_layer_table_operand (const aspen_layer_t *L)
{
    const unsigned int *p = L->params;
    if (L->type != CONV_LAYER && L->type != FC_LAYER && L->type != MATMUL_LAYER) return 0;
    if (aspen_layer_dense3 (L)) return 0;
    return (L->type == MATMUL_LAYER ? p[MAT_K] : p[IN_C]) % 32 != 0;
}

/* A convolution / FC layer whose K axis is laid out as (channel block of 32, tap, channel in block) on the device: every
   layer the kernels read with the stepping loader, i.e. channel count a multiple of 32 and more than one tap (with one
   tap the two orders are the same). */
int aspen_layer_block_major_k (const aspen_layer_t *L)
{
    const unsigned int *p = L->params;
    if (L->type != CONV_LAYER && L->type != FC_LAYER) return 0;
    if (aspen_layer_dense3 (L) || p[IN_C] % 32 != 0) return 0;
    return (L->type == CONV_LAYER ? p[WEIGHT_H] * p[WEIGHT_W] : p[IN_H] * p[IN_W]) > 1;
}

/* padded K of the device layout / 32 (must agree with aspen_layer_to_device) */
unsigned int aspen_layer_kiters (const aspen_layer_t *L)
{
    const unsigned int *p = L->params;
    unsigned int taps, ic;
    if (L->type == CONV_LAYER) { taps = p[WEIGHT_H] * p[WEIGHT_W]; ic = p[IN_C]; }
    else if (L->type == FC_LAYER) { taps = p[IN_H] * p[IN_W]; ic = p[IN_C]; }
    else if (L->type == MATMUL_LAYER) { taps = 1; ic = p[MAT_K]; }
    else return 0;
    if (aspen_layer_dense3 (L)) return round_up (taps * 3, 32) / 32;
    return round_up (taps * round_up (ic, 4), 32) / 32;
}

/* Uploads weight / bias / k-chunk table of one layer for a parent whose column stride is parent_ld
   floats.  Idempotent; re-run after the weights changed. */
int aspen_layer_to_device (aspen_layer_t *L, unsigned int parent_ld)
{
    if (L->type == YOLO_LAYER)
    {
        /* the anchor boxes travel in the weight slot of the device descriptor */
        if (L->d_weight == NULL && (L->d_weight = aspen_hip_alloc (8 * sizeof (float))) == NULL) return -1;
        return aspen_hip_h2d (L->d_weight, L->anchors, 6 * sizeof (float));
    }
    if (L->weight.data == NULL) return 0;
    if (L->d_weight != NULL && L->dev_in_ld == parent_ld) return 0;
    invalidate_device (L);
    const unsigned int *p = L->params;
    if (L->type == LAYERNORM_LAYER)
    {
        L->d_weight = aspen_hip_alloc (L->gemm_m * sizeof (float));
        L->d_bias = aspen_hip_alloc (L->gemm_m * sizeof (float));
        if (!L->d_weight || !L->d_bias) return -1;
        L->dev_in_ld = parent_ld;
        return aspen_hip_h2d (L->d_weight, L->weight.data, L->gemm_m * sizeof (float))
            || aspen_hip_h2d (L->d_bias, L->bias.data, L->gemm_m * sizeof (float));
    }
    unsigned int taps, ic, kw_count, in_w;
    if (L->type == CONV_LAYER) { taps = p[WEIGHT_H] * p[WEIGHT_W]; ic = p[IN_C]; kw_count = p[WEIGHT_W]; in_w = p[IN_W]; }
    else if (L->type == FC_LAYER) { taps = p[IN_H] * p[IN_W]; ic = p[IN_C]; kw_count = p[IN_W]; in_w = p[IN_W]; }
    else { taps = 1; ic = p[MAT_K]; kw_count = 1; in_w = 1; }
    const int dense3 = aspen_layer_dense3 (L);
    const unsigned int icp = dense3 ? 3 : round_up (ic, 4);
    const unsigned int kp = round_up (taps * icp, 32);
    const unsigned int mp = round_up (L->gemm_m, 128);
    float *staged = calloc ((size_t)mp * kp, sizeof (float));
    if (staged == NULL) return -1;
    /* K order on the device.  Channel counts that are multiples of the K slice width: (channel block of 32, tap, channel
       in block), the order the kernels' stepping loader walks (consecutive slices are the taps of one channel block, whose
       windows overlap in the caches).  Otherwise the reference's (tap, channel), each tap's run padded to icp. */
    const int block_major = aspen_layer_block_major_k (L);
    for (unsigned int m = 0; m < L->gemm_m; m++)
        for (unsigned int t = 0; t < taps; t++)
        {
            const float *src = L->weight.data + (size_t)m * L->gemm_k + (size_t)t * ic;
            if (!block_major) memcpy (staged + (size_t)m * kp + (size_t)t * icp, src, ic * sizeof (float));
            else
                for (unsigned int c = 0; c < ic; c += 32)
                    memcpy (staged + (size_t)m * kp + ((size_t)(c / 32) * taps + t) * 32, src + c, 32 * sizeof (float));
        }
    L->d_weight = aspen_hip_alloc ((size_t)mp * kp * sizeof (float));
    int rc = L->d_weight ? aspen_hip_h2d (L->d_weight, staged, (size_t)mp * kp * sizeof (float)) : -1;
    free (staged);
    if (rc) return rc;
    L->d_bias = aspen_hip_alloc (L->gemm_m * sizeof (float));
    if (!L->d_bias || aspen_hip_h2d (L->d_bias, L->bias.data, L->gemm_m * sizeof (float))) return -1;
    if (dense3)
    {
        /* two entries per chunk: K positions [4c, 4c+4) lie in tap 4c / 3 and the tap after it; the entries point at
           the first channel of the two pixels */
        aspen_hip_ktab_t *tab2 = calloc (kp / 2, sizeof (aspen_hip_ktab_t));
        if (tab2 == NULL) return -1;
        for (unsigned int c = 0; c < kp / 4; c++)
            for (unsigned int e = 0; e < 2; e++)
            {
                const unsigned int tap = (c * 4) / 3 + e;
                aspen_hip_ktab_t *t = &tab2[2 * c + e];
                if (tap >= taps) { t->offset = 0; t->kh = 0x4000; t->kw = 0; continue; }
                const unsigned int kh = tap / kw_count, kw = tap % kw_count;
                t->offset = (int32_t)((kh * in_w + kw) * parent_ld);
                t->kh = (uint16_t)kh; t->kw = (uint16_t)kw;
            }
        L->d_ktab = aspen_hip_alloc (kp / 2 * sizeof (aspen_hip_ktab_t));
        rc = L->d_ktab ? aspen_hip_h2d (L->d_ktab, tab2, kp / 2 * sizeof (aspen_hip_ktab_t)) : -1;
        free (tab2);
        L->dev_kp = kp; L->dev_icp = icp; L->dev_in_ld = parent_ld;
        return rc;
    }
    /* k-chunk table: chunk c covers K positions [4c, 4c+4) = tap (4c / icp), channels (4c % icp).. */
    aspen_hip_ktab_t *tab = calloc (kp / 4, sizeof (aspen_hip_ktab_t));
    if (tab == NULL) return -1;
    for (unsigned int c = 0; c < kp / 4; c++)
    {
        const unsigned int tap = (c * 4) / icp, ch = (c * 4) % icp;
        if (tap >= taps) { tab[c].offset = 0; tab[c].kh = 0x4000; tab[c].kw = 0; continue; }
        const unsigned int kh = tap / kw_count, kw = tap % kw_count;
        tab[c].offset = (int32_t)((kh * in_w + kw) * parent_ld + ch);
        tab[c].kh = (uint16_t)kh; tab[c].kw = (uint16_t)kw;
    }
    L->d_ktab = aspen_hip_alloc (kp / 4 * sizeof (aspen_hip_ktab_t));
    rc = L->d_ktab ? aspen_hip_h2d (L->d_ktab, tab, kp / 4 * sizeof (aspen_hip_ktab_t)) : -1;
    free (tab);
    L->dev_kp = kp; L->dev_icp = icp; L->dev_in_ld = parent_ld;
    return rc;
}

/* The device buffers of a matmul layer L that absorbs the layer norm `norm` in front of it (y = W LN (x) + b with
   LN (x) = (x - mean) * rstd * gamma + beta, reference tiled_layernorm, src/tiled_kernels.c:743-782):
     y[m] = rstd * (sum_k W[m][k] gamma[k] x[k]  -  mean * sum_k W[m][k] gamma[k])  +  (b[m] + sum_k W[m][k] beta[k]),
   i.e. the product of the scaled weights with the RAW column, corrected with the column's statistics and the scaled
   weights' row sums.  Sums in double.  Idempotent; dropped with the layer's other device buffers. */
int aspen_layer_norm_fold_to_device (aspen_layer_t *L, const aspen_layer_t *norm)
{
    if (L->d_weight_ln != NULL) return 0;
    if (L->type != MATMUL_LAYER || norm->type != LAYERNORM_LAYER || L->weight.data == NULL || norm->weight.data == NULL
        || norm->gemm_m != L->gemm_k) return -1;
    const unsigned int M = L->gemm_m, K = L->gemm_k, kp = round_up (K, 32), mp = round_up (M, 128);
    float *staged = calloc ((size_t)mp * kp, sizeof (float)), *bias = calloc (M, sizeof (float)), *rowsum = calloc (M, sizeof (float));
    int rc = -1;
    if (staged != NULL && bias != NULL && rowsum != NULL)
    {
        const float *gamma = norm->weight.data, *beta = norm->bias.data;
        for (unsigned int m = 0; m < M; m++)
        {
            const float *w = L->weight.data + (size_t)m * K;
            double rs = 0.0, sh = 0.0;
            for (unsigned int k = 0; k < K; k++)
            {
                const float scaled = w[k] * gamma[k];
                staged[(size_t)m * kp + k] = scaled;
                rs += (double)scaled;
                if (beta != NULL) sh += (double)w[k] * (double)beta[k];
            }
            rowsum[m] = (float)rs;
            bias[m] = (float)((L->bias.data != NULL ? (double)L->bias.data[m] : 0.0) + sh);
        }
        L->d_weight_ln = aspen_hip_alloc ((size_t)mp * kp * sizeof (float));
        L->d_bias_ln = aspen_hip_alloc (M * sizeof (float));
        L->d_rowsum_ln = aspen_hip_alloc (M * sizeof (float));
        if (L->d_weight_ln && L->d_bias_ln && L->d_rowsum_ln)
            rc = aspen_hip_h2d (L->d_weight_ln, staged, (size_t)mp * kp * sizeof (float))
                || aspen_hip_h2d (L->d_bias_ln, bias, M * sizeof (float)) || aspen_hip_h2d (L->d_rowsum_ln, rowsum, M * sizeof (float));
    }
    free (staged); free (bias); free (rowsum);
    return rc;
}
