/* ext.c -- include/aspen_ext.h: mode selection, graph introspection, run statistics, dumps. */
#include "internal.h"
#include "aspen_ext.h"

unsigned int aspen_rpool_num_ninst (rpool_t *rp);
void aspen_nasm_tile_range_internal (const nasm_ldata_t *ld, unsigned int t, unsigned int *r);

void aspen_dse_group_set_mode (dse_group_t *g, int mode) { if (g) g->mode = mode < 0 || mode > 2 ? 2 : mode; }
int aspen_dse_group_last_mode (dse_group_t *g) { return g ? g->last_mode : -1; }
int aspen_dse_group_last_run_ordered (dse_group_t *g)
{
    return g != NULL && g->last_mode == 1 && g->rpool != NULL && g->rpool->graph != NULL && aspen_hip_graph_last_run_ordered (g->rpool->graph);
}
void aspen_nasm_set_ordered (nasm_t *nasm, int ordered)
{
    if (nasm == NULL) return;
    nasm->ordered_pref = ordered < 0 ? -1 : ordered != 0;
    if (nasm->rpool != NULL) nasm->rpool->graph_dirty = 1;        /* the pool's device graph carries the setting: rebuilt at the next run */
}
void aspen_dse_group_set_spin_limit (dse_group_t *g, uint64_t polls) { if (g) g->spin_limit = polls; }
void aspen_dse_group_set_workgroups (dse_group_t *g, unsigned int w) { if (g) g->workgroups = w; }

static int keep_layer_outputs = -1;          /* -1: not set yet, take the environment's word */
void aspen_keep_layer_outputs (int keep) { keep_layer_outputs = keep ? 1 : 0; }
int aspen_keep_layer_outputs_enabled (void)
{
    if (keep_layer_outputs < 0)
    {
        const char *e = getenv ("ASPEN_GPU_KEEP_LAYER_OUTPUTS");
        keep_layer_outputs = e != NULL && atoi (e) != 0;
    }
    return keep_layer_outputs;
}
unsigned int aspen_nasm_num_ldata (nasm_t *n) { return n ? n->num_ldata : 0; }
unsigned int aspen_nasm_num_ninst (nasm_t *n) { return n ? n->num_ninst : 0; }
unsigned int aspen_nasm_num_edges (nasm_t *n) { return n ? n->num_edges : 0; }
uint64_t aspen_nasm_total_flops (nasm_t *n) { return n ? n->total_flops : 0; }
uint64_t aspen_nasm_ldata_flops (nasm_t *n, unsigned int l) { return (n && l < n->num_ldata) ? n->ldata_arr[l].flops : 0; }

void aspen_nasm_ldata_info (nasm_t *n, unsigned int l, unsigned int *info)
{
    if (n == NULL || l >= n->num_ldata || info == NULL) return;
    const nasm_ldata_t *ld = &n->ldata_arr[l];
    info[0] = ld->layer->type; info[1] = ld->layer->activation;
    info[2] = ld->out_mat_dims[OUT_H]; info[3] = ld->out_mat_dims[OUT_W]; info[4] = ld->out_mat_stride;
    info[5] = ld->num_ninst; info[6] = ld->tile_dims[OUT_H]; info[7] = ld->tile_dims[OUT_W];
    info[8] = (unsigned int)ld->parent_ldata_idx[PARENT_0]; info[9] = (unsigned int)ld->parent_ldata_idx[PARENT_1];
    info[10] = ld->ninst_start; info[11] = (unsigned int)ld->variant;
    info[12] = (unsigned int)ld->fused_into; info[13] = (unsigned int)ld->fused_residual;
    info[14] = ld->splits; info[15] = ld->tiles_h; info[16] = ld->kiters_per_split;
    info[17] = (unsigned int)ld->out_discarded; info[18] = (unsigned int)ld->fused_attention; info[19] = (unsigned int)ld->folded_norm;
}

void aspen_nasm_graph (nasm_t *n, const uint32_t **ninst_ldata, const uint32_t **num_parents,
    const uint32_t **child_off, const uint32_t **child_idx)
{
    if (n == NULL) return;
    if (ninst_ldata) *ninst_ldata = n->ninst_ldata;
    if (num_parents) *num_parents = n->num_parents;
    if (child_off) *child_off = n->child_off;
    if (child_idx) *child_idx = n->child_idx;
}

void aspen_nasm_tile_range (nasm_t *n, unsigned int id, unsigned int *range)
{
    if (n == NULL || id >= n->num_ninst || range == NULL) return;
    const nasm_ldata_t *ld = &n->ldata_arr[n->ninst_ldata[id]];
    aspen_nasm_tile_range_internal (ld, id - ld->ninst_start, range);
}

int aspen_rpool_run_stats (rpool_t *rp, uint32_t *executed, uint32_t *double_runs, uint32_t *aborted)
{
    if (rp == NULL || rp->graph == NULL) return -1;
    return aspen_hip_dataflow_stats (rp->graph, executed, double_runs, aborted);
}

int aspen_rpool_profile_layers (rpool_t *rp, unsigned int iters, float *ms)
{
    if (rp == NULL || rp->graph == NULL) return -1;
    return aspen_hip_profile_layers (rp->graph, iters, ms);
}

int aspen_rpool_dataflow_profile (rpool_t *rp, uint64_t ticks[16], int reset)
{
    if (rp == NULL || rp->graph == NULL) return -1;
    return aspen_hip_dataflow_profile (rp->graph, ticks, reset);
}

int aspen_rpool_dataflow_trace (rpool_t *rp, uint64_t *start_end)
{
    if (rp == NULL || rp->graph == NULL) return -1;
    return aspen_hip_dataflow_trace (rp->graph, start_end, aspen_rpool_num_ninst (rp));
}

int aspen_rpool_dataflow_trace_phases (rpool_t *rp, uint64_t *kloop_epilogue)
{
    if (rp == NULL || rp->graph == NULL) return -1;
    return aspen_hip_dataflow_trace_phases (rp->graph, kloop_epilogue, aspen_rpool_num_ninst (rp));
}

int aspen_rpool_debug_set_epoch (rpool_t *rp, uint32_t epoch)
{
    if (rp == NULL || rp->graph == NULL) return -1;
    aspen_hip_graph_debug_set_epoch (rp->graph, epoch);
    return 0;
}

unsigned int aspen_dnn_device_generation (aspen_dnn_t *dnn) { return dnn ? dnn->dev_generation : 0; }

unsigned int aspen_rpool_num_ninst (rpool_t *rp)
{
    unsigned int n = 0;
    if (rp) for (unsigned int i = 0; i < rp->num_nasms; i++) n += rp->nasms[i]->num_ninst;
    return n;
}

/* ---- dumps (reference include/aspen.h:124-133) -------------------------------------------------- */
void print_aspen_build_info (void)
{
    printf ("ASPEN for AMD Instinct MI355X (gfx950): HIP tile kernels + device-side dataflow engine\n");
}

void print_tensor_info (aspen_tensor_t *t, int print_data)
{
    if (t == NULL) { printf ("\t\tTensor: NULL\n"); return; }
    printf ("\t\tNum Elements: %zu\n", t->num_elements);
    if (print_data && t->data)
    {
        for (size_t i = 0; i < t->num_elements; i++) printf ("%s%3.3e ", i % 8 == 0 ? "\n\t\t\t" : "", t->data[i]);
        printf ("\n");
    }
}

void print_layer_info (aspen_layer_t *L, int print_data)
{
    if (L == NULL) { printf ("Error: layer is NULL.\n"); return; }
    printf ("\tLayer %u: %s, activation %s, parents %d %d\n", L->layer_idx, layer_type_str[L->type],
        activation_type_str[L->activation], L->parent_idx[PARENT_0], L->parent_idx[PARENT_1]);
    printf ("\t\tout C/H/W %u/%u/%u  in C/H/W %u/%u/%u  kernel %ux%u stride %u pad %u  M/K %u/%u heads %u\n",
        L->params[OUT_C], L->params[OUT_H], L->params[OUT_W], L->params[IN_C], L->params[IN_H], L->params[IN_W],
        L->params[WEIGHT_H], L->params[WEIGHT_W], L->params[STRIDE], L->params[PADDING],
        L->params[MAT_M], L->params[MAT_K], L->params[NUM_HEAD]);
    if (L->weight.data) { printf ("\t\tWeight [%u][%u]\n", L->gemm_m, L->gemm_k); print_tensor_info (&L->weight, print_data); }
    if (L->bias.data) { printf ("\t\tBias [%u]\n", L->gemm_m); print_tensor_info (&L->bias, print_data); }
}

void print_dnn_info (aspen_dnn_t *dnn, int print_data)
{
    if (dnn == NULL) { printf ("Error: DNN is NULL.\n"); return; }
    printf ("//////// Printing DNN Info ////////\nDNN Name: %s\nNumber of layers: %u\nNumber of nasms: %u\n",
        dnn->name, dnn->num_layers, dnn->ref_nasms);
    for (unsigned int i = 0; i < dnn->num_layers; i++) print_layer_info (&dnn->layers[i], print_data);
}

void print_ldata_info (nasm_ldata_t *ld, int print_ninst, int print_data)
{
    (void)print_data;
    if (ld == NULL) { printf ("Error: ldata is NULL.\n"); return; }
    printf ("\tLdata %u (%s): matrix %u rows x %u columns, stride %u, tiles %u x %u of %u x %u, %u ninsts from %u, %.3f GFLOP\n",
        ld->layer->layer_idx, layer_type_str[ld->layer->type], ld->out_mat_dims[OUT_H], ld->out_mat_dims[OUT_W],
        ld->out_mat_stride, ld->tiles_h, ld->tiles_w, ld->tile_dims[OUT_H], ld->tile_dims[OUT_W], ld->num_ninst,
        ld->ninst_start, (double)ld->flops * 1e-9);
    if (print_ninst)
        for (unsigned int t = 0; t < ld->num_ninst; t++)
        {
            unsigned int r[4];
            aspen_nasm_tile_range_internal (ld, t, r);
            const uint32_t id = ld->ninst_start + t;
            printf ("\t\tNinst %u: columns [%u,%u) rows [%u,%u), %u parents, %u children\n", id, r[0], r[1], r[2], r[3],
                ld->nasm->num_parents[id], ld->nasm->child_off[id + 1] - ld->nasm->child_off[id]);
        }
}

void print_nasm_info (nasm_t *nasm, int print_ninst, int print_data)
{
    if (nasm == NULL) { printf ("Error: nasm is NULL.\n"); return; }
    printf ("//////// Printing NASM Info ////////\nNasm %u of %s: batch %u, seq %u, %u ldata, %u ninsts, %u edges, %.3f GFLOP\n",
        nasm->nasm_id, nasm->dnn->name, nasm->batch_size, nasm->tr_seq_len, nasm->num_ldata, nasm->num_ninst,
        nasm->num_edges, (double)nasm->total_flops * 1e-9);
    for (unsigned int l = 0; l < nasm->num_ldata; l++) print_ldata_info (&nasm->ldata_arr[l], print_ninst, print_data);
}

void print_ninst_info (ninst_t *ninst, int print_data)
{
    (void)ninst; (void)print_data;
    printf ("Tiles are implicit (layer, index) pairs in this build; use print_nasm_info (nasm, 1, 0).\n");
}

void print_rpool_queue_info (rpool_queue_t *q) { (void)q; printf ("The ready queue lives on the device; see print_rpool_info.\n"); }
void print_rpool_queue_group_info (rpool_queue_group_t *q) { (void)q; printf ("The ready queue lives on the device; see print_rpool_info.\n"); }

void print_rpool_info (rpool_t *rp)
{
    if (rp == NULL) { printf ("Error: rpool is NULL.\n"); return; }
    printf ("//////// Printing Ready Pool Info ////////\nAttached nasms: %u, referencing dses: %u, tiles in the merged graph: %u\n",
        rp->num_nasms, rp->ref_dses, aspen_rpool_num_ninst (rp));
    for (unsigned int i = 0; i < rp->num_nasms; i++)
        printf ("\tnasm %u (%s): %u ninsts, %s\n", rp->nasms[i]->nasm_id, rp->nasms[i]->dnn->name, rp->nasms[i]->num_ninst,
            rp->nasms[i]->completed == 1 ? "completed" : rp->nasms[i]->completed == 2 ? "in flight" : rp->nasms[i]->completed == 3 ? "failed" : rp->nasms[i]->armed ? "armed" : "idle");
}
