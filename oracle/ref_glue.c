/*
 * ref_glue.c -- TEST INFRASTRUCTURE ONLY.
 *
 * Thin driver around the *unmodified* reference sources (compiled where they
 * lie under /root/reference by oracle/Makefile into oracle/_ref/).  It lets
 * Python (ctypes) run the reference's own tile kernels layer by layer and read
 * every layer's out_mat, which a normal reference run frees as soon as the
 * consumers finish (reference src/dse.c:84-92).
 *
 * What is called in the reference:
 *   apu_create_dnn                                   src/apu.c:6
 *   apu_create_nasm_without_finding_ninst_parents    src/apu_nasm.c:490
 *   ninst_find_input_pos_idx                         src/apu_nasm.c:37
 *   alloc_ldata_out_mat / copy_buffer_to_ldata_out_mat / copy_ldata_out_mat_to_buffer
 *                                                    src/apu_nasm.c:871 / :809 / :790
 *   tiled_* (the hot path itself)                    src/tiled_kernels.c
 *   dispatch table identical to                      src/dse.c:39-79
 *
 * Edge discovery (ninst_find_parent, minutes at batch 32) is skipped: tiles of
 * one layer are independent, so a layer-synchronous sweep gives the same
 * numbers as the dataflow run.
 *
 * Nothing in the product library links or loads this file.
 */
#include "aspen.h"
#include "apu.h"
#include "nasm.h"
#include "dse.h"
#include "kernels.h"
#include <omp.h>

void ninst_find_input_pos_idx (ninst_t *ninst);

typedef struct
{
    aspen_dnn_t *dnn;
    nasm_t *nasm;
    int num_threads;
    dse_t *dses;
} refglue_t;

static void run_ninst (ninst_t *ninst, dse_t *dse)
{
    switch (ninst->ldata->layer->type)
    {
        case CONV_LAYER:        tiled_conv2d (ninst, dse); break;
        case MAXPOOL_LAYER:     tiled_maxpool2d (ninst, dse); break;
        case AVGPOOL_LAYER:     tiled_avgpool2d (ninst, dse); break;
        case FC_LAYER:          tiled_fully_connected (ninst, dse); break;
        case RESIDUAL_LAYER:    tiled_residual (ninst, dse); break;
        case SOFTMAX_LAYER:     tiled_softmax (ninst, dse); break;
        case YOLO_LAYER:        tiled_yolo (ninst, dse); break;
        case APPEND_LAYER:      tiled_append (ninst, dse); break;
        case MATMUL_LAYER:      tiled_matmul (ninst, dse); break;
        case LAYERNORM_LAYER:   tiled_layernorm (ninst, dse); break;
        case K_ATTENTION_LAYER: tiled_k_attention (ninst, dse); break;
        case V_ATTENTION_LAYER: tiled_v_attention (ninst, dse); break;
        default: break;
    }
}

void *refglue_open (char *cfg_path, char *weight_path, unsigned int batch, unsigned int seq,
    unsigned int min_ninst_per_ldata, int num_threads)
{
    refglue_t *g = calloc (1, sizeof (refglue_t));
    g->dnn = apu_create_dnn (cfg_path, weight_path);
    if (g->dnn == NULL)
    {
        free (g);
        return NULL;
    }
    g->nasm = apu_create_nasm_without_finding_ninst_parents
        (g->dnn, APU_GENERATION_NUM_FLOPS, batch, min_ninst_per_ldata, seq);
    for (unsigned int i = 0; i < g->nasm->num_ninst; i++)
        ninst_find_input_pos_idx (&g->nasm->ninst_arr[i]);
    if (num_threads < 1)
        num_threads = 1;
    g->num_threads = num_threads;
    g->dses = calloc (num_threads, sizeof (dse_t));
    for (int i = 0; i < num_threads; i++)
        g->dses[i].scratchpad = aspen_calloc (DSE_SCRATCHPAD_SIZE, 1);
    for (unsigned int l = 0; l < g->nasm->num_ldata; l++)
        alloc_ldata_out_mat (&g->nasm->ldata_arr[l]);
    return g;
}

int refglue_num_layers (void *h)
{
    return ((refglue_t*)h)->nasm->num_ldata;
}

int refglue_num_ninst (void *h)
{
    return ((refglue_t*)h)->nasm->num_ninst;
}

/* info[0..9] = type, activation, H, W, stride, num_ninst, tile_H, tile_W, parent0, parent1 */
void refglue_layer_info (void *h, int l, unsigned int *info)
{
    nasm_ldata_t *ld = &((refglue_t*)h)->nasm->ldata_arr[l];
    info[0] = ld->layer->type;
    info[1] = ld->layer->activation;
    info[2] = ld->out_mat_dims[OUT_H];
    info[3] = ld->out_mat_dims[OUT_W];
    info[4] = ld->out_mat_stride;
    info[5] = ld->num_ninst;
    info[6] = ld->ninst_tile_dims[OUT_H];
    info[7] = ld->ninst_tile_dims[OUT_W];
    info[8] = ld->parent_ldata_idx_arr[PARENT_0];
    info[9] = ld->parent_ldata_idx_arr[PARENT_1];
}

/* Dense input: W columns of H floats (NHWC for images, [B][S][M] for transformers),
   the layout rpool_add_nasm_raw_input takes (src/rpool.c:167, src/apu_nasm.c:809). */
void refglue_set_input (void *h, float *dense)
{
    refglue_t *g = h;
    copy_buffer_to_ldata_out_mat (&g->nasm->ldata_arr[0], dense);
}

void refglue_forward (void *h)
{
    refglue_t *g = h;
    for (unsigned int l = 1; l < g->nasm->num_ldata; l++)
    {
        nasm_ldata_t *ld = &g->nasm->ldata_arr[l];
        #pragma omp parallel for schedule(dynamic, 1) num_threads(g->num_threads)
        for (int j = 0; j < (int)ld->num_ninst; j++)
            run_ninst (&ld->ninst_arr_start[j], &g->dses[omp_get_thread_num ()]);
    }
}

/* Dense copy of layer l: W columns of H floats, stride padding stripped. */
void refglue_layer_copy (void *h, int l, float *dst)
{
    refglue_t *g = h;
    copy_ldata_out_mat_to_buffer (&g->nasm->ldata_arr[l], dst);
}

double refglue_time_forward (void *h, int iters)
{
    double t0 = omp_get_wtime ();
    for (int i = 0; i < iters; i++)
        refglue_forward (h);
    return (omp_get_wtime () - t0) / iters;
}

/* Packed weight tensor of layer l as the reference holds it after apu_create_dnn
   (src/apu.c:14-40); returns element count, copies at most max_elems floats. */
long refglue_layer_weight (void *h, int l, int tensor_type, float *dst, long max_elems)
{
    refglue_t *g = h;
    aspen_tensor_t *t = g->dnn->layers[l].tensors[tensor_type];
    if (t == NULL)
        return 0;
    long n = t->num_elements;
    if (dst != NULL)
        memcpy (dst, t->data, (n < max_elems ? n : max_elems) * sizeof (float));
    return n;
}

/* Final result through the reference's own unpacker (src/dse.c:515, src/apu.c:227). */
long refglue_result (void *h, int l, int *order, int num_order, float *dst, long max_bytes)
{
    refglue_t *g = h;
    LAYER_PARAMS ord[MAX_TENSOR_DIMS];
    for (int i = 0; i < num_order; i++)
        ord[i] = order[i];
    void *out = NULL;
    ssize_t sz = dse_get_ldata_result (g->nasm, l, ord, &out);
    if (sz > 0 && dst != NULL)
        memcpy (dst, out, sz < max_bytes ? sz : max_bytes);
    free (out);
    return sz;
}

/* the reference's own container writers, for fixtures: the model as a .aspen file, and a .nasm file of
   a graph built with the reference's full tile-dependency search */
void refglue_save_dnn (void *h, char *path)
{
    apu_save_dnn_to_file (((refglue_t*)h)->dnn, path);
}

int refglue_save_nasm (void *h, unsigned int batch, unsigned int seq, unsigned int min_ninst_per_ldata, char *path)
{
    refglue_t *g = h;
    nasm_t *nasm = seq ? apu_create_transformer_nasm (g->dnn, min_ninst_per_ldata, batch, seq)
                       : apu_create_nasm (g->dnn, min_ninst_per_ldata, batch);
    if (nasm == NULL)
        return -1;
    apu_save_nasm_to_file (nasm, path);
    int n = nasm->num_ninst;
    apu_destroy_nasm (nasm);
    return n;
}

/* The reference's own run loop (main.c:105-123) with its own scheduler: a graph with the full tile-dependency
   search (apu_create_nasm: seconds at batch 1, minutes at batch 32), num_dse DSE pthreads on one ready pool,
   `warmup` + `iters` times { rpool_reset_queue; rpool_reset_nasm; dse_group_run; dse_wait_for_nasm_completion;
   dse_group_stop }.  Returns seconds per iteration (< 0 on failure); the final layer of the last iteration goes to
   `result` (dense, W columns of H floats, at most max_floats) through dse_get_nasm_result when result != NULL. */
double refglue_time_dse (void *h, unsigned int batch, unsigned int seq, unsigned int min_ninst_per_ldata, float *dense_input,
    int num_dse, int warmup, int iters, float *result, long max_floats)
{
    refglue_t *g = h;
    nasm_t *nasm = seq ? apu_create_transformer_nasm (g->dnn, min_ninst_per_ldata, batch, seq)
                       : apu_create_nasm (g->dnn, min_ninst_per_ldata, batch);
    if (nasm == NULL)
        return -1.0;
    rpool_t *rpool = rpool_init ();
    dse_group_t *dse_group = dse_group_init (num_dse);
    dse_group_set_rpool (dse_group, rpool);
    rpool_add_nasm_raw_input (rpool, nasm, dense_input);
    double t0 = 0.0;
    for (int i = 0; i < warmup + iters; i++)
    {
        if (i == warmup)
            t0 = omp_get_wtime ();
        if (i > 0)
        {
            rpool_reset_queue (rpool);
            rpool_reset_nasm (rpool, nasm);
        }
        dse_group_run (dse_group);
        dse_wait_for_nasm_completion (nasm);
        dse_group_stop (dse_group);
    }
    const double sec = (omp_get_wtime () - t0) / (iters > 0 ? iters : 1);
    if (result != NULL)
    {
        nasm_ldata_t *last = &nasm->ldata_arr[nasm->num_ldata - 1];
        const long n = (long)last->out_mat_dims[OUT_H] * last->out_mat_dims[OUT_W];
        if (n <= max_floats && last->out_mat != NULL)
            copy_ldata_out_mat_to_buffer (last, result);
    }
    dse_group_destroy (dse_group);
    rpool_destroy (rpool);
    apu_destroy_nasm (nasm);
    return sec;
}

void refglue_close (void *h)
{
    refglue_t *g = h;
    for (int i = 0; i < g->num_threads; i++)
        aspen_free (g->dses[i].scratchpad);
    free (g->dses);
    apu_destroy_nasm (g->nasm);
    apu_destroy_dnn (g->dnn);
    free (g);
}
