/*
 * internal.h -- data model of the C host library behind include/aspen.h.
 *
 * The reference keeps the same three levels (reference include/apu.h:14-43, include/nasm.h:7-66):
 * dnn (layers + weights), nasm (per-layer runtime data + tiles), ninst (one tile).  The layouts
 * here are this library's own: activations live in one device arena per nasm, tiles are implicit
 * (layer, index) pairs, and dependencies are flat CSR arrays ready for upload.
 */
#ifndef ASPEN_AMD_INTERNAL_H
#define ASPEN_AMD_INTERNAL_H

#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "aspen.h"
#include "aspen_hip.h"

#undef ERROR_PRTF     /* the library's own messages carry file and line also under SUPPRESS_OUTPUT */
#define ERROR_PRTF(...) do { fprintf (stderr, "\033[0;31m(%s:%d) ", __FILE__, __LINE__); fprintf (stderr, __VA_ARGS__); fprintf (stderr, "\033[0m"); } while (0)

struct aspen_tensor_t
{
    size_t num_elements;
    float *data;
};

struct aspen_layer_t
{
    aspen_dnn_t *dnn;
    unsigned int layer_idx;
    LAYER_TYPE type;
    LAYER_ACT activation;
    int parent_idx[NUM_PARENT_ELEMENTS];     /* layer index or -1 */
    unsigned int params[NUM_PARAM_ELEMENTS];
    /* host weights in GEMM order: [M][K], K = (kh, kw, ic) for conv, (h, w, c) for FC, plain for
       matmul (the reference's K order, src/apu.c:16,25,34, without its 8-row interleave) */
    aspen_tensor_t weight, bias;
    unsigned int gemm_m, gemm_k;              /* rows / contraction length of `weight` */
    float anchors[6];                         /* YOLO layers: (width, height) of the layer's three anchor boxes */
    /* device copies, created on first use */
    float *d_weight, *d_bias;
    aspen_hip_ktab_t *d_ktab;
    /* matmul layers whose parent is a layer norm that the engine folds into them (see fold_layernorms in nasm.c):
       weights with the norm's scale multiplied into their K axis, bias plus the weights applied to the norm's shift,
       and the row sums of the scaled weights */
    float *d_weight_ln, *d_bias_ln, *d_rowsum_ln;
    unsigned int dev_kp, dev_icp, dev_in_ld;  /* padded K, padded channels per tap, parent stride assumed */
};

struct aspen_dnn_t
{
    char name[MAX_STRING_LEN];
    unsigned int element_size;
    aspen_layer_t *layers;
    unsigned int num_layers;
    unsigned int ref_nasms;
    /* grows whenever a layer's device buffers (weights, bias, k-chunk table) are released: a device graph
       built before that holds stale pointers and is rebuilt before the next run, see dse_group_run */
    unsigned int dev_generation;
};

struct nasm_ldata_t
{
    nasm_t *nasm;
    aspen_layer_t *layer;
    int parent_ldata_idx[NUM_PARENT_ELEMENTS];
    unsigned int out_mat_dims[2];            /* [OUT_W] columns, [OUT_H] rows */
    unsigned int out_mat_stride;
    size_t out_mat_offset;                   /* floats from the start of the arena */
    unsigned int tile_dims[2];
    unsigned int tiles_w, tiles_h;
    unsigned int num_ninst, ninst_start;
    int out_discarded;                       /* fused producer whose own (pre-shortcut) matrix is not written */
    /* split-K: a contraction layer with too few output tiles cuts its K axis into `splits` slices;
       the T*splits tiles (T = tiles_w*tiles_h; index tile*splits + slice) each write one partial product,
       and the one of a group that finishes last sums the slices, adds the bias and activates */
    unsigned int splits, kiters_per_split;
    size_t partial_offset;                   /* floats into the arena: [splits][columns][stride] */
    int variant;
    /* shortcut fusion: a residual layer whose first parent is a contraction layer that feeds nothing
       else is computed in that layer's epilogue (the contraction tile writes its own matrix AND the
       residual's); the residual then owns no tiles.  -1 = not fused */
    int fused_residual;                      /* contraction layer: index of the residual it also produces */
    int fused_into;                          /* residual layer: index of the contraction layer producing it */
    /* attention fusion: a V-attention layer whose K-attention parent feeds nothing else computes scores, exponentials and
       weighted values in one tile (the S x S probabilities stay on chip); the K-attention layer then owns no tiles and
       its matrix is not written.  -1 = not fused */
    int fused_attention;                     /* V-attention layer: index of the K-attention layer it absorbs */
    /* layer-norm folding (fold_layernorms in nasm.c): the matmul layers behind a layer norm take the norm's INPUT and
       normalise it themselves (column statistics gathered in their K loops); the norm then owns no tiles and its matrix
       is not written.  -1 = not folded */
    int folded_norm;                         /* matmul layer: index of the layer norm it absorbs */
    /* a folded norm whose matrix a fused shortcut reads as well: that shortcut's producer normalises the norm's input
       itself, with the column statistics the row-0 tiles of ONE folding layer (stats_writer) store at stats_offset */
    int stats_writer;                        /* layer norm: index of the folding layer that stores the statistics, -1 = none needed */
    size_t stats_offset;                     /* floats into the arena: [columns][2] */
    uint64_t flops;                          /* 2*M*N*K for contraction layers, 64-bit */
};

struct nasm_t
{
    unsigned int nasm_id;
    aspen_dnn_t *dnn;
    unsigned int batch_size, tr_seq_len, min_ninst_per_ldata;
    int preferred_mode;                      /* engine mode the timing tuner found fastest for this graph (0 / 1), -1: not tuned */
    unsigned int kiters_cap;                 /* 0, or the longest K loop (in slices of 32) a contraction tile may have, see create_nasm */
    int small_tiles_only;                    /* every contraction layer uses the small tile shape, see create_nasm */
    int narrow_tiles;                        /* layers short of tiles use the 32 x 32 shape, see create_nasm */
    int ordered_pref;                        /* persistent kernel in its ordered mode (no ready queue): 1 yes (graphs bound by latency, see create_nasm;
                                                the tuner; aspen_nasm_set_ordered), 0 no, -1 the engine decides from the graph's parallelism */
    nasm_ldata_t *ldata_arr;
    unsigned int num_ldata;
    unsigned int num_ninst;
    uint64_t total_flops;
    /* dependency graph over tiles (CSR) */
    uint32_t *ninst_ldata;                   /* tile -> ldata index */
    uint32_t *num_parents;
    uint32_t *child_off, *child_idx;
    uint32_t num_edges;
    /* device state */
    size_t arena_floats;
    float *d_arena;
    rpool_t *rpool;                          /* pool this nasm is attached to */
    unsigned int pool_slot;                  /* its number among the pool's nasms in the merged device graph (aspen_hip_layer_t.graph_id) */
    int armed;                               /* input present and counters to be re-armed at the next run */
    int completed;                           /* 0 not run, 1 completed, 2 in flight, 3 the run failed (stall, launch error) */
};

#define RPOOL_MAX_NASMS 64
struct rpool_t
{
    nasm_t *nasms[RPOOL_MAX_NASMS];
    unsigned int num_nasms;
    unsigned int ref_dses;
    aspen_hip_graph_t *graph;                /* merged device graph of all attached nasms */
    int graph_dirty;
    uint64_t graph_generation;               /* sum of the attached models' dev_generation when the graph was built */
    int running;
};

struct dse_group_t
{
    unsigned int num_dses;
    rpool_t *rpool;
    int mode;                                /* 0 = one launch per layer, 1 = persistent dataflow kernel, 2 = chosen per graph */
    int last_mode;                           /* what the last dse_group_run used (0 / 1) */
    uint64_t spin_limit;                     /* watchdog of the persistent kernel, 0 = default */
    unsigned int workgroups;
};

/* cfg.c */
aspen_dnn_t *aspen_parse_cfg (const char *path);
int aspen_layer_validate (aspen_dnn_t *dnn, aspen_layer_t *layer);
/* dnn.c */
int aspen_layer_to_device (aspen_layer_t *layer, unsigned int parent_ld);
int aspen_load_weight_file (aspen_dnn_t *dnn, const char *path);
int aspen_layer_norm_fold_to_device (aspen_layer_t *L, const aspen_layer_t *norm);
int aspen_layer_dense3 (const aspen_layer_t *layer);            /* three input channels: dense K axis on the device */
int aspen_layer_table_operand (const aspen_layer_t *layer);     /* K axis through the k-chunk table: 64 x 64 tiles only */
int aspen_layer_block_major_k (const aspen_layer_t *layer);     /* device K order (channel block, tap, channel in block) */
unsigned int aspen_layer_kiters (const aspen_layer_t *layer);   /* K slices of 32 of a contraction layer's device layout */
/* nasm.c */
int aspen_nasm_to_device (nasm_t *nasm);
int aspen_nasm_fill_device_layers (nasm_t *nasm, aspen_hip_layer_t *dst, uint32_t ninst_base, uint32_t graph_id);
unsigned int aspen_ld_for_rows (unsigned int rows);

int aspen_keep_layer_outputs_enabled (void);   /* ext.c: see aspen_keep_layer_outputs */

#endif
