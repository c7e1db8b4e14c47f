/*
 * aspen_hip.h -- flat C ABI of the gfx950 tile kernels and the device-side dataflow engine.
 *
 * This is the boundary the C host library (and any other host runtime) binds: plain pointers,
 * sizes and POD descriptors, no C++ or framework types.  It replaces the reference's internal
 * kernel seam
 *     void tiled_X (ninst_t *ninst, dse_t *dse)          reference include/kernels.h:35-46
 *     switch (layer->type) in dse_schedule               reference src/dse.c:39-79
 *     SGEMM_KERNEL* (M,N,K,A,lda,B,ldb,C,ldc)            reference include/kernels.h:15-33
 * and the scheduler / ready-pool protocol around it
 *     dse_schedule, update_children_*                    reference src/dse.c:20-108, :363-401
 *     rpool_push_ninsts / rpool_fetch_ninsts             reference src/rpool.c:611-685
 *     push_first_layer_to_rpool                          reference src/dse.c:443-470
 *
 * Data contract (same as the reference's out_mat, reference src/apu_nasm.c:950-1017):
 * an activation is a matrix of N columns x M rows stored column by column with a stride of `ld`
 * floats (NHWC with a padded channel run).  Padding rows [M, ld) are zero and are never written.
 * All pointers inside aspen_hip_layer_t are DEVICE pointers obtained from aspen_hip_alloc.
 *
 * Every function returns 0 on success and a non-zero HIP error code otherwise (the text is
 * available from aspen_hip_last_error); allocation returns NULL on failure.
 */
#ifndef ASPEN_AMD_ASPEN_HIP_H
#define ASPEN_AMD_ASPEN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* One k-chunk (4 consecutive floats of the implicit-GEMM K axis) of a conv / FC layer:
   where it sits relative to the top-left input pixel of an output position. */
typedef struct aspen_hip_ktab_t
{
    int32_t offset;      /* (kh*IW + kw)*ld_in + ic, in floats */
    uint16_t kh, kw;     /* tap; kh >= 0x4000 marks a chunk beyond the real K (reads as zero) */
} aspen_hip_ktab_t;

/* aspen_hip_layer_t.direct.  TABLE: K order (tap, channel padded to 4), one table entry per k-chunk.  DIRECT: the
   parent's columns are the K axis.  DENSE3: a convolution over 3 input channels with K order (tap, channel) and NO
   padding (weights [roundup(M,128)][Kp], Kp = roundup(3 * taps, 32) <= 512): k-chunk c = K positions 4c .. 4c+3 covers
   the last 3 - c % 3 channels of tap 4c / 3 and the first c % 3 + 1 of the next tap; the table holds TWO entries per
   chunk, 2c for the first tap and 2c + 1 for the second, each with the offset of that pixel's channel 0. */
enum { ASPEN_HIP_OPERAND_TABLE = 0, ASPEN_HIP_OPERAND_DIRECT = 1, ASPEN_HIP_OPERAND_DENSE3 = 2 };
/* aspen_hip_layer_t.direct of a V-attention layer.  FUSED: the layer's tiles compute the scores, their exponentials
   and the weighted values in one pass from in0 = Query, in1 = Key and fuse_in = Value (stride fuse_ld_in), with
   `masked` as the K-attention layer has it; the K-attention layer in front of it then has no tiles and its S x S
   matrix is not written (one head of hd <= 64, hd % 32 == 0, channels per tile).  0: in0 = probabilities, in1 = Value. */
enum { ASPEN_HIP_ATTENTION_FUSED = 1 };

/* GEMM tile shapes (rows of the weight matrix x activation columns per workgroup): LARGE = the
   biggest shape of the build (128 x 64 by default), WIDE = 64 x 128, SMALL = 64 x 64, NARROW = 32 x 32 with the
   workgroup's four wavefronts splitting the K axis (for graphs bound by the latency of their dependency
   chains; operands DIRECT or TABLE with IC % 32 == 0 only), TALL = 128 x 32 for layers that stream a large weight
   matrix past at most 32 columns (fully connected layers at small batch; not with the k-chunk table of a channel
   count off the slice width, nor DENSE3).  SMALL, NARROW and TALL tiles may be cut along K (splits).  The graph
   builder asks aspen_hip_tile_shapes for the numbers instead of assuming them. */
enum { ASPEN_HIP_GEMM_LARGE = 0, ASPEN_HIP_GEMM_WIDE = 1, ASPEN_HIP_GEMM_SMALL = 2, ASPEN_HIP_GEMM_NARROW = 3, ASPEN_HIP_GEMM_TALL = 4, ASPEN_HIP_NUM_GEMM_VARIANTS };
/* shapes[2*v] = rows, shapes[2*v+1] = columns of GEMM variant v = 0..2; shapes[6] = queries per K-attention
   tile; shapes[7] = queries per V-attention tile; shapes[8] = workgroups per compute unit the
   kernels are built for; shapes[9], shapes[10] = rows, columns of variant 3; shapes[11], shapes[12] = of variant 4.  Pure
   constants: callable without a GPU. */
void aspen_hip_tile_shapes (uint32_t shapes[13]);

/* Per-layer descriptor: everything one tile needs, so a tile is (layer, tile index).
   Replaces the fields the reference's tiled_* read through ninst->ldata->layer
   (reference include/nasm.h:28-66, include/apu.h:33-43). */
typedef struct aspen_hip_layer_t
{
    int32_t type;            /* LAYER_TYPE of aspen.h */
    int32_t act;             /* LAYER_ACT of aspen.h */
    int32_t variant;         /* GEMM tile shape for contraction layers */
    int32_t direct;          /* how the B operand is found, ASPEN_HIP_OPERAND_*: 0 k-chunk table, 1 read in place (1x1 stride-1
                                conv / matmul, K % 32 == 0), 2 dense three-channel table */
    uint32_t M, N, ld;       /* output rows, columns, stride */
    uint32_t tile_m, tile_n; /* tile extent in rows / columns: the GEMM variant's shape; an uncut (splits == 1) layer of the LARGE
                                shape may also have tile_m = 2 or 4 times the shape's rows (one workgroup runs those row tiles of
                                its column block one after the other) */
    uint32_t tiles_m, tiles_n;
    uint32_t ninst_start;    /* engine-wide index of this layer's first tile */
    uint32_t num_ninst;
    uint32_t K, Kp;          /* contraction length, padded to a multiple of 32 */
    uint32_t ld0, ld1;       /* strides of the parents */
    uint32_t IH, IW, IC, OH, OW, KH, KW, stride, pad;
    uint32_t heads, seq, hd, masked;
    /* split-K (contraction layers): the layer has T*splits tiles, T = tiles_m*tiles_n; tile
       (tile*splits + slice) computes the partial products over kiters_per_split K slices and writes
       them to `partial` ([splits][T] blocks of tile_m*tile_n floats in the kernel's own register order;
       64 x 64 and 32 x 32 tiles only).  The `splits` tiles of one output tile form a group: the
       member that finishes last (an arrival counter decides) sums the slices in slice order, adds
       the bias, activates and writes the output; only it releases the group's children */
    uint32_t splits, kiters_per_split;
    uint32_t fuse_discard;   /* 1 (only with fuse_out): the layer's own, pre-shortcut matrix `out` is not written */
    /* 1 (matmul layers with a DIRECT operand, 64 x 64 tiles, K axis not cut, K a multiple of 32): a layer norm over the
       K axis of the operand is folded into the layer (reference tiled_layernorm, src/tiled_kernels.c:743-782, eps 1e-6):
       in0 is the norm's INPUT, `weight` holds W[m][k] * gamma[k], `bias` b[m] + sum_k W[m][k] * beta[k], in1 the row sums
       of `weight` ([M]); a tile gathers sum and sum of squares of its columns in its K loop and computes
       out = act (rstd[n] * (acc[m][n] - mean[n] * in1[m]) + bias[m]) */
    uint32_t norm_fold;
    uint32_t reserved0;
    /* Where the folded norm's matrix is still needed as a fused shortcut's operand (a post-norm transformer block), nobody
       writes it either: the tiles of row 0 of ONE of the folding layers store their columns' mean and
       1 / sqrt (variance + eps) to norm_stats ([N][2] floats; NULL: not stored), and the layer with the fused shortcut
       gets the norm's INPUT as fuse_in together with fuse_norm_stats (those pairs), fuse_norm_gamma and
       fuse_norm_beta ([M]; beta may be NULL): its epilogue normalises the operand piece by piece,
       (x - mean[n]) * rstd[n] * gamma[m] + beta[m], before it adds it.  fuse_norm_stats == NULL: fuse_in is used as it
       is.  64 x 64 tiles over a multiple of 64 channels only. */
    float *norm_stats;
    const float *fuse_norm_stats, *fuse_norm_gamma, *fuse_norm_beta;
    uint32_t graph_id;       /* which of the co-scheduled networks of one engine run the layer belongs to (0 .. 63): the run
                                reports each network's completion separately, see aspen_hip_graph_group_done */
    float *partial;
    float *out;
    const float *in0;        /* PARENT_0 */
    const float *in1;        /* PARENT_1 */
    const float *weight;     /* [roundup(M,128)][Kp] row-major, zero padded; layernorm: gamma[M].  K order of a convolution /
                                FC operand that is neither DIRECT nor DENSE3: IC % 32 == 0 (the kernels step through it):
                                (channel block of 32, kh, kw, channel in block); else (kh, kw, channel padded to 4), the
                                order the k-chunk table describes */
    const float *bias;       /* [M] or NULL */
    const aspen_hip_ktab_t *ktab; /* Kp/4 entries (Kp/2 for DENSE3), NULL when direct */
    /* fused shortcut (contraction layers; reference tiled_residual, src/tiled_kernels.c:613-638, run in
       the epilogue): besides out = act(...) the tile also writes
       fuse_out = fuse_act (out + fuse_in) at the same rows / columns; fuse_out has stride ld.
       fuse_out == NULL: no fusion.  The residual layer itself then has num_ninst == 0. */
    float *fuse_out;
    const float *fuse_in;
    uint32_t fuse_ld_in;
    int32_t fuse_act;
    /* Derived values, filled in by aspen_hip_graph_create (callers leave them zero): divisions by OH*OW, OW,
       tiles_m and splits as multiply-and-shift pairs {multiplier, shift} (a tile's set-up is bound by
       instruction issue, and an integer division costs some 25 instructions), and the number of columns of
       the first parent's matrix. */
    uint32_t div_ohw[2], div_ow[2], div_tiles_m[2], div_splits[2];
    uint32_t in0_columns;
} aspen_hip_layer_t;

typedef struct aspen_hip_graph_t aspen_hip_graph_t;

/* ---- device, memory, transfers --------------------------------------------------------------- */
int aspen_hip_init (void);
const char *aspen_hip_last_error (void);
/* compute units, engine clock (kHz), HBM bytes, device name */
int aspen_hip_device_info (int *num_cu, int *clock_khz, size_t *mem_bytes, char *name, int name_len);
void *aspen_hip_alloc (size_t bytes);            /* zero-filled device memory */
void aspen_hip_free (void *ptr);
int aspen_hip_h2d (void *dst, const void *src, size_t bytes);
int aspen_hip_d2h (void *dst, const void *src, size_t bytes);
/* strided copies: `rows` runs of `width` bytes, pitches in bytes */
int aspen_hip_h2d_2d (void *dst, size_t dpitch, const void *src, size_t spitch, size_t width, size_t rows);
int aspen_hip_d2h_2d (void *dst, size_t dpitch, const void *src, size_t spitch, size_t width, size_t rows);
int aspen_hip_zero (void *dst, size_t bytes);
/* dense host matrix (`columns` runs of `rows` floats) -> device matrix with column stride `ld` >= rows floats,
   the padding rows zeroed: one contiguous upload into a staging buffer the library keeps, then a kernel
   that spreads the columns (what the reference's copy_buffer_to_ldata_out_mat, src/apu_nasm.c:809-826, does
   on the host).  dense_device_to_host is the inverse (reference get_packed_ldata_output_colwise). */
int aspen_hip_dense_host_to_device (float *dst, uint32_t ld, const float *src_host, uint32_t rows, size_t columns);
int aspen_hip_dense_device_to_host (float *dst_host, const float *src, uint32_t ld, uint32_t rows, size_t columns);
/* device-to-device copy by a plain streaming kernel on the library's stream (asynchronous); size and
   addresses multiples of 16 bytes.  Its memory traffic is exactly 2 x bytes, which makes it the
   calibration point for a profiler's HBM byte counters. */
int aspen_hip_copy (void *dst, const void *src, size_t bytes);

/* ---- graph ----------------------------------------------------------------------------------- */
/* Uploads a tile graph.  ninst_layer[i] = layer of tile i; num_parents[i] = its dependency count;
   children of tile i are child_idx[child_off[i] .. child_off[i+1]).  roots = tiles with no parent
   left once the input layer counts as complete.  The members of a split-K group (see
   aspen_hip_layer_t.splits) all carry the same child list, and a child counts the whole group as
   ONE parent: whichever member finishes last releases it.  (reference: ninst_t, include/nasm.h:50-66) */
aspen_hip_graph_t *aspen_hip_graph_create (const aspen_hip_layer_t *layers, uint32_t num_layers,
    const uint32_t *ninst_layer, const uint32_t *num_parents, const uint32_t *child_off,
    const uint32_t *child_idx, uint32_t num_ninst, const uint32_t *roots, uint32_t num_roots);
void aspen_hip_graph_destroy (aspen_hip_graph_t *graph);
/* Average parallelism of the uploaded graph: summed tile cost over the cost of the longest dependency
   chain (cost = K slices of a contraction tile plus a constant).  The default grid of a dataflow run
   is sized from it; a host runtime can use it to prefer one launch per layer for graphs that could
   never keep a persistent grid busy (a single image through a deep network). */
double aspen_hip_graph_parallelism (const aspen_hip_graph_t *graph);

/* ---- execution (all asynchronous on the library's stream) -------------------------------------- */
/* One launch per layer, layers [first, last] in index order: the per-operator baseline and the
   per-kernel profiling mode. */
int aspen_hip_run_layers (aspen_hip_graph_t *graph, uint32_t first_layer, uint32_t last_layer);
/* Barrier-free execution: re-arms the dependency counters and the ready queue, then one persistent
   kernel of `workgroups` workgroups (0 = a whole number per compute unit, 1 to 4, sized from the graph's
   average parallelism) pops ready tiles until all are done.
   spin_limit bounds every wait on the ready queue (0 = default); a wait that exceeds it raises the
   abort flag of THIS graph, all workgroups exit and aspen_hip_graph_sync (graph) returns ASPEN_HIP_ERR_STALLED. */
int aspen_hip_run_dataflow (aspen_hip_graph_t *graph, uint32_t workgroups, uint64_t spin_limit);
#define ASPEN_HIP_ERR_STALLED 0x7001
/* Debug switches for later dataflow runs.  SKIP_TILES runs the whole dependency protocol with empty
   tiles: the scheduler-only mode of the reference (-D_SKIP_KERNELS=1, reference src/tiled_kernels.c:163). */
#define ASPEN_HIP_FLAG_SKIP_TILES 1u
/* COUNT_TILES keeps the per-tile execution counters that aspen_hip_dataflow_stats reports (one extra
   pair of atomics per tile); without it `executed` and `double_runs` read 0. */
#define ASPEN_HIP_FLAG_COUNT_TILES 2u
/* PROFILE makes every workgroup of the dataflow kernel accumulate where its time went. */
#define ASPEN_HIP_FLAG_PROFILE 4u
/* ticks (100 MHz) summed over all workgroups since the last reset: [0] inside tiles, [1] waiting for
   the tile's stores to be acknowledged, [2] scheduling step (publish, pop, waiting for a ready tile),
   [3] total workgroup lifetime; detail of [2]: [4] publishing wavefront (countdown of the children,
   pushes), [5] popping wavefront drawing its ticket, [6] popping wavefront waiting for its queue slot
   to be filled; [7] engine-clock cycles of the workgroups' lifetimes ([7] / [3] x 100 MHz = the
   average engine clock during the run); contraction tiles only: [12] descriptor and operand-address set-up, [8] from
   there to the first staged slice (the first loads' latency), [9] K loop, [10] epilogue, [11] split-K arrival
   and reduction; [13..15] unused */
int aspen_hip_dataflow_profile (aspen_hip_graph_t *graph, uint64_t ticks[16], int reset);
/* TRACE makes the dataflow kernel stamp every tile's start and end (100 MHz device clock);
   aspen_hip_dataflow_trace copies the stamps of the last traced run: start_end[2*i], [2*i+1] for tile i
   of the graph's num_ninst tiles. */
#define ASPEN_HIP_FLAG_TRACE 8u
/* NO_HANDOFF sends every tile that becomes ready through the queue, instead of letting the workgroup that
   finished its last parent run it next (for comparisons). */
#define ASPEN_HIP_FLAG_NO_HANDOFF 16u
/* XCD_QUEUES gives every XCD a ready queue of its own and every tile a home XCD (a fixed eighth of its layer's
   columns), so that tiles reading the same activations share an L2: about 40 % less memory traffic on the
   convolutional networks, but free workgroups cannot help another XCD and runs take 0-11 % longer.  Also switched on
   by ASPEN_GPU_XCD_QUEUES in the environment; ASPEN_GPU_XCD_QUEUE_SHIFT = 1 / 2 groups the XCDs in pairs / fours (4 / 2
   queues).  Needs a grid that is a multiple of 8 workgroups (else ignored).  Without the flag a run whose grid fills the
   device takes TWO queues (one per half of the XCDs: same run time as one queue, a tenth less memory traffic) and every
   other run one; ASPEN_GPU_XCD_QUEUES=0 forces one queue everywhere. */
#define ASPEN_HIP_FLAG_XCD_QUEUES 32u
/* ORDERED / NO_ORDERED force or forbid the ordered mode of the persistent kernel, which a run otherwise takes when
   the graph's average parallelism is below 128 tiles (one image through a deep network): no ready queue; workgroups
   take the tiles in index order (parents first), prepare each one and request its first weights before it is ready,
   then wait on the tile's own dependency counter.  Also ASPEN_GPU_ORDERED=0|1 in the environment. */
void aspen_hip_graph_set_ordered (aspen_hip_graph_t *graph, int ordered);     /* 1 / 0: this graph's dataflow runs use / do not use the ordered mode; -1: decided from its parallelism */
int aspen_hip_graph_last_run_ordered (const aspen_hip_graph_t *graph);          /* 1 when the graph's last dataflow run was an ordered one */
#define ASPEN_HIP_FLAG_ORDERED 64u
#define ASPEN_HIP_FLAG_NO_ORDERED 128u
int aspen_hip_dataflow_trace (aspen_hip_graph_t *graph, uint64_t *start_end, uint32_t num_ninst);
/* Two more stamps per contraction tile of the same traced run: kloop_epilogue[2*i] = end of tile i's K loop,
   [2*i+1] = its epilogue's (or, for a split-K member, its partial sums') stores issued; 0 for other tiles. */
int aspen_hip_dataflow_trace_phases (aspen_hip_graph_t *graph, uint64_t *kloop_epilogue, uint32_t num_ninst);
void aspen_hip_set_flags (uint32_t flags);
/* Waits for everything enqueued on the library's stream.  Reports device errors only; whether a dataflow
   run was given up is a property of its graph, see aspen_hip_graph_sync. */
int aspen_hip_sync (void);
/* aspen_hip_sync, then ASPEN_HIP_ERR_STALLED if the last dataflow run of `graph` was given up by its
   watchdog (the flag is consumed).  A stall of one graph is never reported against another. */
int aspen_hip_graph_sync (aspen_hip_graph_t *graph);
/* 1 when everything enqueued so far has finished, 0 when still running */
int aspen_hip_idle (void);
/* Completion of ONE of the networks co-scheduled in a dataflow run (the layers with graph_id == group), the
   counterpart of the reference marking a nasm completed when its own last layer has finished while other
   nasms are still running (reference src/dse.c:94-105, waiter :279-289).  The tile that finishes a network
   (its last tile without children) raises a pinned host word, so neither call touches the stream.
   group_done: 1 = finished in the graph's last dataflow run, 0 = not yet, -1 = unknown (no such group, or the
   last run was one launch per layer: ask aspen_hip_idle / aspen_hip_graph_sync).
   wait_group blocks until the group has finished, the whole run has ended, or the run was given up; it returns 0,
   or -1 for an unknown group (the caller still learns of a stalled run from aspen_hip_graph_sync). */
int aspen_hip_graph_group_done (aspen_hip_graph_t *graph, uint32_t group);
int aspen_hip_graph_wait_group (aspen_hip_graph_t *graph, uint32_t group);
/* aspen_hip_d2h on a second stream: does not wait for work enqueued on the library's main stream, so a network
   that has finished can be read out while the persistent kernel still runs the others.  Only memory whose
   producers have finished may be read this way (tiles write through to memory before they are published). */
int aspen_hip_d2h_side (void *dst, const void *src, size_t bytes);
/* Test hook: sets the tag the graph's next dataflow run derives its queue-entry tag from (tags cycle through
   1 .. 65535 and the queues are cleared when they wrap). */
void aspen_hip_graph_debug_set_epoch (aspen_hip_graph_t *graph, uint32_t epoch);
/* Counters of the last dataflow run (kept under ASPEN_HIP_FLAG_COUNT_TILES): tiles executed, tiles executed
   more than once, and the abort flag.  That no tile starts before its parents have ended is checked from
   the time stamps of a traced run (ASPEN_HIP_FLAG_TRACE), not counted on the device. */
int aspen_hip_dataflow_stats (aspen_hip_graph_t *graph, uint32_t *executed, uint32_t *double_runs, uint32_t *abort_flag);

/* ---- timing ------------------------------------------------------------------------------------- */
/* Average duration of each layer's kernel over `iters` back-to-back launches (HIP events around the
   launches of one layer); ms_per_layer holds one float per layer, 0 for the input layer.  The layers
   run in index order, so the activations are those of a real forward pass. */
int aspen_hip_profile_layers (aspen_hip_graph_t *graph, uint32_t iters, float *ms_per_layer);
/* HIP events on the library's stream: record into slot [0,12), elapsed between two recorded slots.
   Slots 14 and 15 are recorded by aspen_hip_run_dataflow right before and after the persistent
   kernel, so elapsed(14, 15) is that kernel's duration. */
int aspen_hip_event_record (int slot);
int aspen_hip_event_elapsed_ms (int slot_begin, int slot_end, float *ms);

/* {multiplier, shift} with which the kernels divide by `d` (see aspen_hip_layer_t); pure arithmetic, callable
   without a GPU. */
void aspen_hip_divider_for (uint32_t d, uint32_t out[2]);

/* ---- plain SGEMM seam (reference include/kernels.h:15-33 on device pointers) -------------------- */
/* C[n*ldc + m] = act(bias[m] + sum_k A[m*lda + k] * B[n*ldb + k]); A row-major [M][K] (not packed),
   lda/ldb/ldc multiples of 4, K a multiple of 32. */
int aspen_hip_sgemm (uint32_t M, uint32_t N, uint32_t K, const float *A, uint32_t lda, const float *B,
    uint32_t ldb, float *C, uint32_t ldc, const float *bias, int act);

/* The same SGEMM for callers that cannot allocate device memory (tight serving loops, harnesses that forbid
   hipMalloc).  No counterpart in the reference.  It runs on the library's own stream (it cannot be recorded into a
   caller's stream capture) and the first call initialises the library (stream, events, kernel attributes: call
   aspen_hip_init beforehand where that matters).  It calls no hipMalloc / hipFree:
   the zero-padded staging copy of A that aspen_hip_sgemm allocates per call lives in a static device array of
   aspen_hip_sgemm_static_max_bytes () bytes (8 MiB per GPU, held until the process ends), so
   roundup (M, 128) * K * 4 must not exceed that; larger problems are refused with a message.  Asynchronous on
   the library's stream: C is complete after aspen_hip_sync ().  All calls on a GPU share the one staging
   array; the library's stream orders them, calls issued concurrently from several host threads would race. */
int aspen_hip_sgemm_static (uint32_t M, uint32_t N, uint32_t K, const float *A, uint32_t lda, const float *B,
    uint32_t ldb, float *C, uint32_t ldc, const float *bias, int act);
size_t aspen_hip_sgemm_static_max_bytes (void);

#ifdef __cplusplus
}
#endif
#endif /* ASPEN_AMD_ASPEN_HIP_H */
