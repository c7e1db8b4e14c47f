/*
 * aspen_ext.h -- additions to the public API that have no counterpart in the reference: engine mode
 * selection, introspection of the tile graph (used by the tests and the benchmark) and run statistics.
 */
#ifndef ASPEN_AMD_ASPEN_EXT_H
#define ASPEN_AMD_ASPEN_EXT_H

#include <stdint.h>
#include "aspen.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Loads an ASPEN_DATA weight file into an existing model (reference include/apu.h:46, src/apu_file_io.c:48; the
   reference calls it from apu_create_dnn and keeps it out of its public header).  Allowed at any time
   between runs: ready pools that hold a graph of the model pick the new weights up at their next run. */
void apu_load_dnn_data_from_file (aspen_dnn_t *dnn, char *input_path);
/* how often device copies of the model's weights have been released (by a reload); a ready pool compares it
   with the value its device graph was built at */
unsigned int aspen_dnn_device_generation (aspen_dnn_t *dnn);

/* 0: one kernel launch per layer (layer-synchronous); 1: persistent dataflow kernel; 2 (default): the
   persistent kernel, unless the graph came from apu_generate_nasm and its timing found one launch per layer faster.
   The environment variable ASPEN_GPU_MODE=layers|dataflow|auto sets the initial value. */
void aspen_dse_group_set_mode (dse_group_t *dse_group, int mode);
/* the mode the last dse_group_run used: 0 or 1 (-1 before the first run) */
int aspen_dse_group_last_mode (dse_group_t *dse_group);
/* 1 when that run was a dataflow run in ordered mode (tiles taken in index order and prepared before they are ready,
   no ready queue: what graphs built for one image through a deep network run in) */
int aspen_dse_group_last_run_ordered (dse_group_t *dse_group);
/* Whether runs of this nasm on the persistent kernel use its ordered mode (no ready queue; tiles assigned to workgroups in
   index order and prepared before their parents have finished): 1 / 0, -1 = the engine decides.  apu_create_nasm asks
   for it on graphs bound by their dependency chains (convolutional networks at small and medium batches, transformers
   with up to about a thousand tokens), apu_generate_nasm times
   it against the other engines; a pool runs ordered when all its nasms ask for it. */
void aspen_nasm_set_ordered (nasm_t *nasm, int ordered);
/* Watchdog of the persistent kernel: polls a workgroup may spend waiting for one ready tile before the
   run is given up (every workgroup then leaves, the run reports ASPEN_HIP_ERR_STALLED and the next run
   starts from re-armed state).  0 = the library's default (2^26 polls, minutes). */
void aspen_dse_group_set_spin_limit (dse_group_t *dse_group, uint64_t polls);
/* persistent workgroups of the dataflow kernel; 0 = sized from the graph's average parallelism (1 to 4 per compute unit) */
void aspen_dse_group_set_workgroups (dse_group_t *dse_group, unsigned int workgroups);

/* Graphs created AFTER this call keep (1) or do not keep (0, the default) the matrix of a contraction
   layer whose shortcut is computed in its own epilogue.  Nothing on the device reads that matrix, and
   the reference frees a layer's matrix as soon as its children are done (src/dse.c:84-92), so by
   default it is not written; dse_get_ldata_result on such a layer then reports an error.  The
   environment variable ASPEN_GPU_KEEP_LAYER_OUTPUTS=1 sets the initial value. */
void aspen_keep_layer_outputs (int keep);

unsigned int aspen_nasm_num_ldata (nasm_t *nasm);
unsigned int aspen_nasm_num_ninst (nasm_t *nasm);
unsigned int aspen_nasm_num_edges (nasm_t *nasm);
uint64_t aspen_nasm_total_flops (nasm_t *nasm);
/* info[0..19] = type, activation, rows, columns, stride, num_ninst, tile_rows, tile_columns,
   parent0, parent1 (0xffffffff = none), first tile index, GEMM variant,
   [12] shortcut layers: index of the contraction layer whose tiles produce this layer (0xffffffff = own tiles),
   [13] contraction layers: index of the shortcut layer fused into the epilogue (0xffffffff = none),
   [14] split-K slices, [15] row tiles, [16] K slices of 32 per split-K part,
   [17] 1 when the layer's matrix is not written (nothing on the device reads it and outputs are not kept),
   [18] V-attention layers: index of the K-attention layer whose work its tiles absorb (0xffffffff = none), [19] reserved (0) */
void aspen_nasm_ldata_info (nasm_t *nasm, unsigned int ldata_idx, unsigned int *info);
uint64_t aspen_nasm_ldata_flops (nasm_t *nasm, unsigned int ldata_idx);
/* dependency graph in CSR form; pointers stay valid until the nasm is destroyed */
void aspen_nasm_graph (nasm_t *nasm, const uint32_t **ninst_ldata, const uint32_t **num_parents,
    const uint32_t **child_off, const uint32_t **child_idx);
/* column / row range [c0, c1) x [r0, r1) of one tile */
void aspen_nasm_tile_range (nasm_t *nasm, unsigned int ninst_idx, unsigned int *range);

/* counters of the last dataflow run of the pool: tiles executed, tiles executed more than once,
   abort flag (a wait on the ready queue hit its spin limit).  Returns 0 on success. */
int aspen_rpool_run_stats (rpool_t *rpool, uint32_t *executed, uint32_t *double_runs, uint32_t *aborted);
/* per-layer kernel time (ms) of the pool's merged graph in layer-launch mode, averaged over iters;
   ms must hold one float per layer of every attached nasm, in attachment order */
int aspen_rpool_profile_layers (rpool_t *rpool, unsigned int iters, float *ms);
/* where the workgroups of the dataflow kernel spent their time (needs ASPEN_HIP_FLAG_PROFILE) */
int aspen_rpool_dataflow_profile (rpool_t *rpool, uint64_t ticks[16], int reset);
/* start / end time stamps (100 MHz) of every tile of the pool's last run made with ASPEN_HIP_FLAG_TRACE;
   start_end holds 2 * aspen_rpool_num_ninst values, tiles in pool order (nasms in attachment order) */
int aspen_rpool_dataflow_trace (rpool_t *rpool, uint64_t *start_end);
/* the K-loop / epilogue stamps of the same run (aspen_hip_dataflow_trace_phases), same order */
int aspen_rpool_dataflow_trace_phases (rpool_t *rpool, uint64_t *kloop_epilogue);
/* Test hook: the tag the pool's next dataflow run derives its queue-entry tag from (aspen_hip_graph_debug_set_epoch);
   returns -1 when the pool has no device graph yet. */
int aspen_rpool_debug_set_epoch (rpool_t *rpool, uint32_t epoch);
/* tiles in the pool's merged graph */
unsigned int aspen_rpool_num_ninst (rpool_t *rpool);

#ifdef __cplusplus
}
#endif
#endif
