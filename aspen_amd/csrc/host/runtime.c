/*
 * runtime.c -- ready pool, scheduling-engine group and result read-out on top of the device engine.
 *
 * Same call protocol as the reference (reference main.c:105-151):
 *   rpool_init -> dse_group_init -> dse_group_set_rpool -> rpool_add_nasm[_raw_input]
 *   loop { rpool_reset_queue; rpool_reset_nasm; dse_group_run; dse_wait_for_nasm_completion; dse_group_stop }
 *   dse_get_nasm_result
 * The reference's pool of mutex-guarded queues and its DSE pthreads (reference src/rpool.c,
 * src/dse.c) live on the device here: the ready queue and the dependency counters are arrays in
 * HBM and the "engines" are the persistent workgroups of one kernel; this file only arms and
 * launches them.  Every nasm attached to a pool runs in the same launch, its tiles interleaved
 * with the others' in one queue (co-scheduled networks, reference examples/2).
 */
#include "internal.h"

/* ---- ready pool -------------------------------------------------------------------------------- */
rpool_t *rpool_init (void)
{
    rpool_t *rp = calloc (1, sizeof (rpool_t));
    if (rp == NULL) { ERROR_PRTF ("ERROR: rpool_init: out of host memory.\n"); return NULL; }
    rp->graph_dirty = 1;
    return rp;
}

void rpool_destroy (rpool_t *rpool)
{
    if (rpool == NULL) return;
    if (rpool->ref_dses > 0)
    {
        ERROR_PRTF ("Cannot destroy rpool with %u dses still referencing it.\n", rpool->ref_dses);
        return;
    }
    aspen_hip_sync ();
    for (unsigned int i = 0; i < rpool->num_nasms; i++) rpool->nasms[i]->rpool = NULL;
    aspen_hip_graph_destroy (rpool->graph);
    free (rpool);
}

static int attach (rpool_t *rpool, nasm_t *nasm)
{
    if (nasm->rpool == rpool) return 0;
    if (nasm->rpool != NULL) { ERROR_PRTF ("nasm %u is already attached to another rpool\n", nasm->nasm_id); return -1; }
    if (rpool->num_nasms == RPOOL_MAX_NASMS) { ERROR_PRTF ("rpool is full (%d nasms)\n", RPOOL_MAX_NASMS); return -1; }
    rpool->nasms[rpool->num_nasms++] = nasm;
    nasm->rpool = rpool;
    rpool->graph_dirty = 1;
    return 0;
}

void rpool_add_nasm_raw_input (rpool_t *rpool, nasm_t *nasm, void *input_data)
{
    if (rpool == NULL) { ERROR_PRTF ("ERROR: rpool_add_nasm_raw_input: rpool is NULL.\n"); return; }
    if (nasm == NULL) { ERROR_PRTF ("ERROR: rpool_add_nasm_raw_input: nasm is NULL.\n"); return; }
    if (aspen_nasm_to_device (nasm)) { ERROR_PRTF ("ERROR: rpool_add_nasm_raw_input: device setup failed: %s\n", aspen_hip_last_error ()); return; }
    if (attach (rpool, nasm)) return;
    if (input_data != NULL)
    {
        /* dense columns -> strided columns of layer 0 (reference copy_buffer_to_ldata_out_mat, src/apu_nasm.c:809) */
        const nasm_ldata_t *ld = &nasm->ldata_arr[0];
        const size_t H = ld->out_mat_dims[OUT_H], W = ld->out_mat_dims[OUT_W];
        aspen_hip_sync ();
        /* one contiguous transfer, then a kernel that spreads the columns to the matrix's stride: a strided
           copy of millions of 12-byte columns (3-channel images) is orders of magnitude slower, and
           repacking on the host costs more than the transfer */
        const int rc = aspen_hip_dense_host_to_device (nasm->d_arena + ld->out_mat_offset, ld->out_mat_stride, input_data, (uint32_t)H, W);
        if (rc) ERROR_PRTF ("ERROR: rpool_add_nasm_raw_input: input upload failed: %s\n", aspen_hip_last_error ());
    }
    nasm->armed = 1;
    nasm->completed = 0;
}

void rpool_add_nasm (rpool_t *rpool, nasm_t *nasm, char *input_filename)
{
    if (rpool == NULL || nasm == NULL) { ERROR_PRTF ("ERROR: rpool_add_nasm: NULL argument.\n"); return; }
    const nasm_ldata_t *ld = &nasm->ldata_arr[0];
    const unsigned int *p = ld->layer->params;
    const size_t H = ld->out_mat_dims[OUT_H], W = ld->out_mat_dims[OUT_W], n = H * W;
    float *file = calloc (n, sizeof (float)), *dense = calloc (n, sizeof (float));
    if (file == NULL || dense == NULL)
    {
        ERROR_PRTF ("ERROR: rpool_add_nasm: out of host memory.\n");
        free (file); free (dense);
        return;
    }
    if (input_filename != NULL)
    {
        FILE *fp = fopen (input_filename, "rb");
        if (fp == NULL || fread (file, sizeof (float), n, fp) != n)
        {
            ERROR_PRTF ("Error: Failed to read %zu floats from file %s.\n", n, input_filename);
            if (fp) fclose (fp);
            free (file); free (dense);
            return;
        }
        fclose (fp);
    }
    if (nasm->tr_seq_len == 0)
    {
        /* image files are NCHW (reference aspen_load_input_NHWC, src/apu.c:638) */
        const size_t C = p[OUT_C], HW = (size_t)p[OUT_H] * p[OUT_W];
        for (size_t b = 0; b < nasm->batch_size; b++)
            for (size_t c = 0; c < C; c++)
                for (size_t i = 0; i < HW; i++)
                    dense[(b * HW + i) * C + c] = file[(b * C + c) * HW + i];
    }
    else
        memcpy (dense, file, n * sizeof (float));
    rpool_add_nasm_raw_input (rpool, nasm, dense);
    free (file); free (dense);
}

void rpool_reset_queue (rpool_t *rpool)
{
    /* the device queue is rebuilt by the arm kernel of the next run; nothing is kept between runs */
    (void)rpool;
}

void rpool_reset_nasm (rpool_t *rpool, nasm_t *nasm)
{
    if (rpool == NULL || nasm == NULL) return;
    if (nasm->rpool != rpool)
    {
        ERROR_PRTF ("ERROR: rpool_reset_nasm: nasm \"%s_nasm_%d\" is not in rpool.\n", nasm->dnn->name, nasm->nasm_id);
        return;
    }
    apu_reset_nasm (nasm);
}

static uint64_t pool_generation (const rpool_t *rp)
{
    uint64_t g = 0;
    for (unsigned int i = 0; i < rp->num_nasms; i++) g += rp->nasms[i]->dnn->dev_generation;
    return g;
}

/* merged device graph of every nasm in the pool: layer and tile indices shifted, roots interleaved */
static int rebuild_graph (rpool_t *rp)
{
    aspen_hip_sync ();
    aspen_hip_graph_destroy (rp->graph);
    rp->graph = NULL;
    uint32_t layers = 0, ninst = 0, edges = 0;
    for (unsigned int i = 0; i < rp->num_nasms; i++)
    {
        layers += rp->nasms[i]->num_ldata; ninst += rp->nasms[i]->num_ninst; edges += rp->nasms[i]->num_edges;
    }
    if (layers == 0) { rp->graph_dirty = 0; return 0; }
    aspen_hip_layer_t *L = calloc (layers, sizeof (aspen_hip_layer_t));
    uint32_t *nl = calloc (ninst + 1, sizeof (uint32_t)), *np = calloc (ninst + 1, sizeof (uint32_t));
    uint32_t *co = calloc ((size_t)ninst + 2, sizeof (uint32_t)), *ci = calloc (edges + 1, sizeof (uint32_t));
    uint32_t *roots = calloc (ninst + 1, sizeof (uint32_t));
    uint32_t lbase = 0, nbase = 0, ebase = 0, nroots = 0;
    int rc = 0;
    if (L == NULL || nl == NULL || np == NULL || co == NULL || ci == NULL || roots == NULL)
    {
        ERROR_PRTF ("ERROR: out of host memory while merging the graphs of the pool.\n");
        rc = -1;
    }
    for (unsigned int i = 0; i < rp->num_nasms && !rc; i++)
    {
        nasm_t *g = rp->nasms[i];
        if (aspen_nasm_to_device (g)) { rc = -1; break; }
        g->pool_slot = i;
        aspen_nasm_fill_device_layers (g, L + lbase, nbase, i);
        for (uint32_t t = 0; t < g->num_ninst; t++)
        {
            nl[nbase + t] = lbase + g->ninst_ldata[t];
            np[nbase + t] = g->num_parents[t];
            co[nbase + t] = ebase + g->child_off[t];
        }
        for (uint32_t e = 0; e < g->num_edges; e++) ci[ebase + e] = nbase + g->child_idx[e];
        lbase += g->num_ldata; nbase += g->num_ninst; ebase += g->num_edges;
    }
    if (!rc) co[ninst] = edges;
    /* roots of the attached graphs taken in turns, so co-scheduled networks start together */
    if (!rc)
    {
        uint32_t cursor[RPOOL_MAX_NASMS] = {0}, base[RPOOL_MAX_NASMS];
        uint32_t b = 0;
        for (unsigned int i = 0; i < rp->num_nasms; i++) { base[i] = b; b += rp->nasms[i]->num_ninst; }
        int progress = 1;
        while (progress)
        {
            progress = 0;
            for (unsigned int i = 0; i < rp->num_nasms; i++)
            {
                nasm_t *g = rp->nasms[i];
                while (cursor[i] < g->num_ninst && g->num_parents[cursor[i]] != 0) cursor[i]++;
                if (cursor[i] < g->num_ninst) { roots[nroots++] = base[i] + cursor[i]++; progress = 1; }
            }
        }
        rp->graph = aspen_hip_graph_create (L, layers, nl, np, co, ci, ninst, roots, nroots);
        if (rp->graph == NULL) rc = -1;
        else
        {
            /* graphs bound by latency run the persistent kernel in its ordered mode: when every nasm of the pool asks for it;
               a nasm that asks for the ready queue gets it; otherwise the engine decides from the merged graph */
            int all_ordered = rp->num_nasms > 0, any_queue = 0;
            for (unsigned int i = 0; i < rp->num_nasms; i++) { all_ordered &= rp->nasms[i]->ordered_pref == 1; any_queue |= rp->nasms[i]->ordered_pref == 0; }
            if (all_ordered) aspen_hip_graph_set_ordered (rp->graph, 1);
            else if (any_queue) aspen_hip_graph_set_ordered (rp->graph, 0);
        }
    }
    free (L); free (nl); free (np); free (co); free (ci); free (roots);
    rp->graph_dirty = rc != 0;
    rp->graph_generation = pool_generation (rp);
    return rc;
}

/* ---- scheduling engines ------------------------------------------------------------------------ */
dse_group_t *dse_group_init (unsigned int num_dse)
{
    dse_group_t *g = calloc (1, sizeof (dse_group_t));
    if (g == NULL) { ERROR_PRTF ("ERROR: dse_group_init: out of host memory.\n"); return NULL; }
    g->num_dses = num_dse;
    g->mode = 2;
    g->last_mode = -1;
    const char *m = getenv ("ASPEN_GPU_MODE");           /* "layers" = one launch per layer, "dataflow" = persistent kernel, "auto" */
    if (m != NULL && strcmp (m, "layers") == 0) g->mode = 0;
    if (m != NULL && strcmp (m, "dataflow") == 0) g->mode = 1;
    const char *w = getenv ("ASPEN_GPU_WORKGROUPS");
    g->workgroups = w ? (unsigned int)atoi (w) : 0;
    return g;
}

void dse_group_set_rpool (dse_group_t *dse_group, rpool_t *rpool)
{
    if (dse_group == NULL) { ERROR_PRTF ("ERROR: dse_group_set_rpool: dse_group is NULL\n"); return; }
    if (rpool == NULL) { ERROR_PRTF ("ERROR: dse_group_set_rpool: rpool is NULL\n"); return; }
    if (dse_group->rpool != NULL) dse_group->rpool->ref_dses -= dse_group->num_dses;
    dse_group->rpool = rpool;
    rpool->ref_dses += dse_group->num_dses;
}

void dse_group_destroy (dse_group_t *dse_group)
{
    if (dse_group == NULL) return;
    aspen_hip_sync ();
    if (dse_group->rpool != NULL) dse_group->rpool->ref_dses -= dse_group->num_dses;
    free (dse_group);
}

void dse_group_run (dse_group_t *dse_group)
{
    if (dse_group == NULL) { ERROR_PRTF ("ERROR: dse_group_run: dse_group is NULL\n"); return; }
    rpool_t *rp = dse_group->rpool;
    if (rp == NULL) { ERROR_PRTF ("ERROR: dse_group_run: no rpool set\n"); return; }
    int armed = 0;
    for (unsigned int i = 0; i < rp->num_nasms; i++) armed |= rp->nasms[i]->armed;
    if (!armed) return;                                    /* nothing ready: the engines idle, as in the reference */
    /* a model whose weights were loaded again since the graph was built has released the device buffers the
       graph's layer descriptors point to */
    if (rp->graph != NULL && rp->graph_generation != pool_generation (rp)) rp->graph_dirty = 1;
    if (rp->graph_dirty && rebuild_graph (rp)) { ERROR_PRTF ("ERROR: dse_group_run: graph upload failed: %s\n", aspen_hip_last_error ()); return; }
    if (rp->graph == NULL) return;
    int rc;
    /* auto: the persistent kernel (in its ordered mode for graphs built for latency: ResNet-50 batch 1 0.45 ms against
       0.54 ms as one launch per layer), unless the timing tuner found one launch per layer faster for this graph */
    int mode = dse_group->mode;
    if (mode == 2)
    {
        /* graphs the timing tuner produced carry its verdict; it counts when all graphs of the pool agree */
        int tuned = rp->num_nasms ? rp->nasms[0]->preferred_mode : -1;
        for (unsigned int i = 1; i < rp->num_nasms; i++) if (rp->nasms[i]->preferred_mode != tuned) tuned = -1;
        mode = tuned >= 0 ? tuned : 1;
    }
    dse_group->last_mode = mode;
    if (mode == 0)
    {
        uint32_t layers = 0;
        for (unsigned int i = 0; i < rp->num_nasms; i++) layers += rp->nasms[i]->num_ldata;
        rc = aspen_hip_run_layers (rp->graph, 0, layers - 1);
    }
    else
        rc = aspen_hip_run_dataflow (rp->graph, dse_group->workgroups, dse_group->spin_limit);
    if (rc) { ERROR_PRTF ("ERROR: dse_group_run: launch failed: %s\n", aspen_hip_last_error ()); return; }
    for (unsigned int i = 0; i < rp->num_nasms; i++) { rp->nasms[i]->armed = 0; rp->nasms[i]->completed = 2; }   /* 2 = in flight */
    rp->running = 1;
}

static void finish (rpool_t *rp)
{
    if (rp == NULL || !rp->running) return;
    /* a run the device gave up (watchdog, launch error) leaves its graphs NOT completed: 3 = failed */
    int state = 1;
    if (aspen_hip_graph_sync (rp->graph)) { ERROR_PRTF ("ERROR: device run failed: %s\n", aspen_hip_last_error ()); state = 3; }
    rp->running = 0;
    for (unsigned int i = 0; i < rp->num_nasms; i++)
        if (rp->nasms[i]->completed == 2) rp->nasms[i]->completed = state;
}

void dse_group_stop (dse_group_t *dse_group)
{
    if (dse_group == NULL) { ERROR_PRTF ("ERROR: dse_group_stop: dse_group is NULL\n"); return; }
    finish (dse_group->rpool);
}

/* Per-nasm completion (reference src/dse.c:94-105: the thread that finishes a nasm's last layer sets
   nasm->completed and signals that nasm's waiter, whatever the other nasms of the pool are doing; waiter
   :279-289).  In a dataflow run the tile that finishes a nasm raises a host word for it, so a nasm can be
   waited for and read out while the persistent kernel is still working on the others.  One launch per layer
   has no such signal: there a nasm is complete when the stream has drained. */
static int nasm_done_on_device (const nasm_t *nasm)
{
    const rpool_t *rp = nasm->rpool;
    return rp != NULL && rp->running && rp->graph != NULL && aspen_hip_graph_group_done (rp->graph, nasm->pool_slot) == 1;
}

void dse_wait_for_nasm_completion (nasm_t *nasm)
{
    if (nasm == NULL) return;
    if (nasm->completed != 2) return;
    rpool_t *rp = nasm->rpool;
    if (rp != NULL && rp->running && rp->graph != NULL && aspen_hip_graph_wait_group (rp->graph, nasm->pool_slot) == 0 && nasm_done_on_device (nasm))
    {
        nasm->completed = 1;        /* the others stay in flight; dse_group_stop (or a wait for them) drains the run */
        return;
    }
    finish (rp);
}

unsigned int dse_check_nasm_completion (nasm_t *nasm)
{
    if (nasm == NULL) return 0;
    if (nasm->completed == 2)
    {
        if (aspen_hip_idle () == 1) finish (nasm->rpool);
        else if (nasm_done_on_device (nasm)) nasm->completed = 1;
    }
    return nasm->completed == 1;
}

void dse_group_run_until_nasm_completion (dse_group_t *dse_group, nasm_t *nasm)
{
    dse_group_run (dse_group);
    dse_wait_for_nasm_completion (nasm);
    dse_group_stop (dse_group);
}

/* ---- results ------------------------------------------------------------------------------------ */
/* Layer output as a dense tensor in the caller's dimension order (reference get_ldata_output,
   src/apu.c:227-297): stride padding stripped, native order (batch, positions..., channels) permuted. */
static ssize_t get_ldata_output (nasm_t *nasm, unsigned int ldata_idx, LAYER_PARAMS *order, void **out_ptr);

/* For a YOLO layer the reference returns ALL detection heads of the network, concatenated per image
   in layer order (reference src/dse.c:472-513); so does this function when a dimension order is given.
   order == NULL (an extension) always returns the one layer's own matrix as [columns][rows]. */
ssize_t dse_get_ldata_result (nasm_t *nasm, unsigned int ldata_idx, LAYER_PARAMS *order, void **out_ptr)
{
    if (nasm == NULL || ldata_idx >= nasm->num_ldata) { ERROR_PRTF ("Error in get_ldata_output: ldata is NULL.\n"); return -1; }
    if (order == NULL || nasm->ldata_arr[ldata_idx].layer->type != YOLO_LAYER) return get_ldata_output (nasm, ldata_idx, order, out_ptr);
    if (out_ptr == NULL) { ERROR_PRTF ("Error in get_ldata_output: out_ptr is NULL.\n"); return -1; }
    void *parts[64];
    ssize_t bytes[64], total = 0;
    int n = 0;
    for (unsigned int l = 0; l < nasm->num_ldata && n < 64; l++)
    {
        if (nasm->ldata_arr[l].layer->type != YOLO_LAYER) continue;
        bytes[n] = get_ldata_output (nasm, l, order, &parts[n]);
        if (bytes[n] < 0) { for (int i = 0; i < n; i++) free (parts[i]); return -1; }
        total += bytes[n++];
    }
    char *outp = calloc (total ? (size_t)total : 1, 1);
    if (outp == NULL) { for (int i = 0; i < n; i++) free (parts[i]); return -1; }
    size_t off = 0;
    const size_t B = nasm->batch_size;
    for (size_t b = 0; b < B; b++)
        for (int i = 0; i < n; i++)
        {
            const size_t per = (size_t)bytes[i] / B;
            memcpy (outp + off, (char *)parts[i] + per * b, per);
            off += per;
        }
    for (int i = 0; i < n; i++) free (parts[i]);
    *out_ptr = outp;
    return total;
}

static ssize_t get_ldata_output (nasm_t *nasm, unsigned int ldata_idx, LAYER_PARAMS *order, void **out_ptr)
{
    if (nasm == NULL || ldata_idx >= nasm->num_ldata) { ERROR_PRTF ("Error in get_ldata_output: ldata is NULL.\n"); return -1; }
    if (out_ptr == NULL) { ERROR_PRTF ("Error in get_ldata_output: out_ptr is NULL.\n"); return -1; }
    if (nasm->d_arena == NULL) { ERROR_PRTF ("Error in get_ldata_output: nasm has not been run.\n"); return -1; }
    if (nasm->completed == 2) dse_wait_for_nasm_completion (nasm);
    if (nasm->completed == 3 && ldata_idx != 0)
    {
        ERROR_PRTF ("Error in get_ldata_output: the last run of this nasm failed; its layers hold no valid result.\n");
        return -1;
    }
    const nasm_ldata_t *ld = &nasm->ldata_arr[ldata_idx];
    const aspen_layer_t *L = ld->layer;
    if (ld->out_discarded)
    {
        ERROR_PRTF ("Error in get_ldata_output: layer %u feeds only the shortcut computed in its own epilogue and its matrix was not kept "
                    "(aspen_keep_layer_outputs (1) before creating the nasm keeps it).\n", ldata_idx);
        return -1;
    }
    const size_t H = ld->out_mat_dims[OUT_H], W = ld->out_mat_dims[OUT_W];
    float *dense = malloc (H * W * sizeof (float));
    if (dense == NULL) return -1;
    int rc;
    if (nasm->rpool != NULL && nasm->rpool->running && aspen_hip_idle () != 1)
    {
        /* this nasm has finished but the persistent kernel is still running others: anything enqueued on its stream
           (also the kernel that strips the padding rows) would wait for the whole run.  The matrix is copied as it is
           on a second stream and the padding stripped here. */
        const size_t ldm = ld->out_mat_stride;
        float *raw = ldm == H ? dense : malloc (W * ldm * sizeof (float));
        rc = raw == NULL ? -1 : aspen_hip_d2h_side (raw, nasm->d_arena + ld->out_mat_offset, W * ldm * sizeof (float));
        if (raw != NULL && raw != dense)
        {
            for (size_t c = 0; c < W && !rc; c++) memcpy (dense + c * H, raw + c * ldm, H * sizeof (float));
            free (raw);
        }
    }
    else    /* padding rows stripped on the device, one contiguous transfer */
        rc = aspen_hip_dense_device_to_host (dense, nasm->d_arena + ld->out_mat_offset, ld->out_mat_stride, (uint32_t)H, W);
    if (rc)
    {
        ERROR_PRTF ("Error in get_ldata_output: download failed: %s\n", aspen_hip_last_error ());
        free (dense);
        return -1;
    }
    /* native dimension list, slowest first */
    LAYER_PARAMS native[4];
    size_t dim[NUM_PARAM_ELEMENTS] = {0};
    int nd;
    const unsigned int *p = L->params;
    const int matrix = nasm->tr_seq_len != 0;
    if (L->type == K_ATTENTION_LAYER)
    {
        nd = 4; native[0] = BATCH; native[1] = NUM_HEAD; native[2] = MAT_N; native[3] = MAT_M;
        dim[BATCH] = nasm->batch_size; dim[NUM_HEAD] = p[NUM_HEAD]; dim[MAT_N] = nasm->tr_seq_len; dim[MAT_M] = H;
    }
    else if (matrix)
    {
        nd = 3; native[0] = BATCH; native[1] = MAT_N; native[2] = MAT_M;
        dim[BATCH] = nasm->batch_size; dim[MAT_N] = nasm->tr_seq_len; dim[MAT_M] = H;
    }
    else if (L->type == FC_LAYER || L->type == SOFTMAX_LAYER)
    {
        nd = 2; native[0] = BATCH; native[1] = OUT_C;
        dim[BATCH] = nasm->batch_size; dim[OUT_C] = H;
    }
    else
    {
        nd = 4; native[0] = BATCH; native[1] = OUT_H; native[2] = OUT_W; native[3] = OUT_C;
        dim[BATCH] = nasm->batch_size; dim[OUT_H] = p[OUT_H]; dim[OUT_W] = p[OUT_W]; dim[OUT_C] = H;
    }
    /* the first nd entries of `order` must be a permutation of the native dimensions */
    int valid = order != NULL;
    for (int i = 0; i < nd && valid; i++)
    {
        int found = 0;
        for (int j = 0; j < nd; j++) found |= native[j] == order[i];
        for (int j = 0; j < i; j++) if (order[j] == order[i]) found = 0;
        valid = found;
    }
    if (!valid) { *out_ptr = dense; return (ssize_t)(H * W * sizeof (float)); }   /* native order */
    size_t nstride[NUM_PARAM_ELEMENTS] = {0}, s = 1;
    for (int i = nd - 1; i >= 0; i--) { nstride[native[i]] = s; s *= dim[native[i]]; }
    float *out = calloc (H * W, sizeof (float));
    if (out == NULL) { free (dense); return -1; }
    size_t idx[4] = {0, 0, 0, 0};
    for (size_t o = 0; o < H * W; o++)
    {
        size_t src = 0;
        for (int i = 0; i < nd; i++) src += idx[i] * nstride[order[i]];
        out[o] = dense[src];
        for (int i = nd - 1; i >= 0; i--) { if (++idx[i] < dim[order[i]]) break; idx[i] = 0; }
    }
    free (dense);
    *out_ptr = out;
    return (ssize_t)(H * W * sizeof (float));
}

ssize_t dse_get_nasm_result (nasm_t *nasm, LAYER_PARAMS *order, void **out_ptr)
{
    if (nasm == NULL) return -1;
    return dse_get_ldata_result (nasm, nasm->num_ldata - 1, order, out_ptr);
}

void aspen_flush_dynamic_memory (void)
{
    /* activations live in per-nasm arenas that are freed with the nasm; there is no allocator cache to flush */
}
