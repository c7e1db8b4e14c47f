/*
 * aspen.h -- public C API of the MI355X tiled-dataflow library.
 *
 * Drop-in for the reference's public header (reference include/aspen.h:50-133):
 * same function names, argument meaning and ownership rules; enum numbering is
 * kept because callers pass LAYER_PARAMS arrays (output dimension order) by
 * value.  All structs are opaque here; no caller in the reference touches a
 * field (reference main.c and the examples directory).
 *
 * Each declaration cites the reference declaration it replaces.
 */
#ifndef ASPEN_AMD_ASPEN_H
#define ASPEN_AMD_ASPEN_H

/* System headers a caller gets through the reference header (reference include/aspen.h:4-18) and relies
   on: the reference's main.c and examples include nothing but aspen.h, yet use FILE, printf, strcpy,
   atoi, gettimeofday and friends. */
#ifndef _GNU_SOURCE
#define _GNU_SOURCE
#endif
#include <stddef.h>
#include <string.h>
#include <stdio.h>
#include <stdlib.h>
#include <ctype.h>
#include <math.h>
#include <float.h>
#include <limits.h>
#include <stdint.h>
#include <time.h>
#include <sys/time.h>
#include <sys/types.h>
#include <assert.h>
#include <unistd.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MAX_TENSOR_DIMS 8      /* reference include/aspen.h:26 */
#define MAX_STRING_LEN 256     /* reference include/aspen.h:27 */

/* Console macros of the reference header (reference include/aspen.h:34-48): same names and colours, silenced
   by SUPPRESS_OUTPUT != 0.  No shipped caller uses them; they are here so that code written against the
   reference header compiles unchanged. */
#ifndef SUPPRESS_OUTPUT
#define SUPPRESS_OUTPUT 0
#endif
#define ASPEN_COLOUR_PRTF_(stream, colour, ...) do { fprintf (stream, "\033[0;" colour "m"); fprintf (stream, __VA_ARGS__); fprintf (stream, "\033[0m"); } while (0)
#if SUPPRESS_OUTPUT == 0
#define PRTF(...) printf (__VA_ARGS__)
#define ERROR_PRTF(...) do { fprintf (stderr, "\033[0;31m(%s:%d)", __FILE__, __LINE__); fprintf (stderr, __VA_ARGS__); fprintf (stderr, "\033[0m"); } while (0)
#define RED_PRTF(...) ASPEN_COLOUR_PRTF_ (stdout, "31", __VA_ARGS__)
#define GREEN_PRTF(...) ASPEN_COLOUR_PRTF_ (stdout, "32", __VA_ARGS__)
#define YELLOW_PRTF(...) ASPEN_COLOUR_PRTF_ (stdout, "33", __VA_ARGS__)
#define BLUE_PRTF(...) ASPEN_COLOUR_PRTF_ (stdout, "34", __VA_ARGS__)
#else
#define PRTF(...) ((void)0)
#define ERROR_PRTF(...) fprintf (stderr, "\033[0;31mASPEN: An error has occured.\033[0m")
#define RED_PRTF(...) ((void)0)
#define GREEN_PRTF(...) ((void)0)
#define YELLOW_PRTF(...) ((void)0)
#define BLUE_PRTF(...) ((void)0)
#endif

/* reference include/aspen.h:50 */
typedef enum { NINST_NOT_READY, NINST_READY, NINST_COMPLETED, NUM_NINST_STATES } NINST_STATE;

/* reference include/aspen.h:51-55 */
typedef enum {
    NO_LAYER_TYPE, INPUT_LAYER, CONV_LAYER, FC_LAYER, RESIDUAL_LAYER, BATCHNORM_LAYER, YOLO_LAYER,
    APPEND_LAYER, ACTIVATION_LAYER, MAXPOOL_LAYER, AVGPOOL_LAYER, ROUTE_LAYER, SOFTMAX_LAYER,
    MATMUL_LAYER, LAYERNORM_LAYER, K_ATTENTION_LAYER, V_ATTENTION_LAYER, NUM_LAYER_ELEMENTS
} LAYER_TYPE;

/* reference include/aspen.h:56-60.  OUT_W = 0 and OUT_H = 1 double as indices of
   2-element matrix-dimension arrays (columns, rows). */
typedef enum {
    OUT_W, OUT_H, OUT_C, BATCH, IN_W, IN_H, IN_C, WEIGHT_W, WEIGHT_H, SUB_C, STRIDE, PADDING,
    DILATION, GROUPS, NUM_HIDDEN, NUM_HEAD, NUM_SEQ, MAT_M, MAT_N, MAT_K, SUB_M, MASKED,
    FORM_BYTES, NUM_PARAM_ELEMENTS
} LAYER_PARAMS;

/* reference include/aspen.h:61-62 */
typedef enum {
    NULL_TENSOR, OUTPUT_TENSOR, INPUT_TENSOR, WEIGHT_TENSOR, BIAS_TENSOR, COL_IDX_TENSOR,
    ANCHOR_TENSOR, BN_VAR_TENSOR, BN_MEAN_TENSOR, BN_WEIGHT_TENSOR, NUM_TENSORS
} LAYER_TENSORS;

/* reference include/aspen.h:63 */
typedef enum { PARENT_NONE, PARENT_0, PARENT_1, PARENT_WEIGHT, NUM_PARENT_ELEMENTS } LAYER_PARENTS;

/* reference include/aspen.h:64 */
typedef enum {
    NO_ACTIVATION, SIGMOID, LINEAR, TANH, RELU, LEAKY_RELU, ELU, SELU, GELU, GELU_ACCURATE,
    NUM_ACTIVATIONS
} LAYER_ACT;

/* reference include/aspen.h:65.  Ready-pool routing conditions: kept for source compatibility; this
   library has one device-side ready queue and routes nothing. */
typedef enum { RPOOL_DNN, RPOOL_LAYER_TYPE, RPOOL_LAYER_IDX, RPOOL_NASM, RPOOL_DSE, NUM_RPOOL_CONDS } RPOOL_CONDS;

/* Printable names of the enumerators above, indexed by value (reference include/aspen.h:67-73, tables in
   src/util.c:3-41). */
extern char *ninst_state_str[NUM_NINST_STATES];
extern char *layer_type_str[NUM_LAYER_ELEMENTS];
extern char *param_type_str[NUM_PARAM_ELEMENTS];
extern char *tensor_type_str[NUM_TENSORS];
extern char *parent_type_str[NUM_PARENT_ELEMENTS];
extern char *activation_type_str[NUM_ACTIVATIONS];
extern char *rpool_cond_str[NUM_RPOOL_CONDS];

typedef struct aspen_dnn_t aspen_dnn_t;       /* model: layers + weights          (include/aspen.h:74) */
typedef struct aspen_layer_t aspen_layer_t;
typedef struct aspen_tensor_t aspen_tensor_t;
typedef struct ninst_t ninst_t;               /* one output tile                  (include/aspen.h:78) */
typedef struct nasm_t nasm_t;                 /* tile dependency graph            (include/aspen.h:79) */
typedef struct nasm_ldata_t nasm_ldata_t;     /* per-layer runtime data           (include/aspen.h:80) */
typedef struct rpool_t rpool_t;               /* ready pool                       (include/aspen.h:82) */
typedef struct rpool_queue_t rpool_queue_t;
typedef struct rpool_queue_group_t rpool_queue_group_t;
typedef struct dse_t dse_t;
typedef struct dse_group_t dse_group_t;       /* scheduling engines               (include/aspen.h:87) */

/* ---- model ------------------------------------------------------------------------------- */
/* reference include/aspen.h:90.  cfg = Darknet-style text; data_path = ASPEN_DATA weight file or
   NULL (then weights stay at their seeded-random initial values).  NULL on failure. */
aspen_dnn_t *apu_create_dnn (char *input_path, char *data_path);
/* reference include/aspen.h:91.  Refuses (prints, returns) while nasms still reference the dnn. */
void apu_destroy_dnn (aspen_dnn_t *dnn);
/* reference include/aspen.h:92-93 */
void apu_save_dnn_to_file (aspen_dnn_t *dnn, char *filename);
aspen_dnn_t *apu_load_dnn_from_file (char *filename);

/* ---- graph ------------------------------------------------------------------------------- */
/* reference include/aspen.h:95-96: tile-size search by timing the engine. */
nasm_t *apu_generate_nasm (aspen_dnn_t *dnn, unsigned int batch_size, unsigned int num_iter);
nasm_t *apu_generate_transformer_nasm (aspen_dnn_t *dnn, unsigned int batch_size, unsigned int seq_num, unsigned int num_iter);
/* reference include/aspen.h:97-98 */
nasm_t *apu_create_nasm (aspen_dnn_t *dnn, unsigned int min_ninst_per_ldata, unsigned int batch_size);
nasm_t *apu_create_transformer_nasm (aspen_dnn_t *dnn, unsigned int min_ninst_per_ldata, unsigned int batch_size, unsigned int seq_num);
/* reference include/aspen.h:99-102 */
void apu_destroy_nasm (nasm_t *nasm);
nasm_t *apu_load_nasm_from_file (char *filename, aspen_dnn_t *dnn);
void apu_save_nasm_to_file (nasm_t *nasm, char *filename);
void apu_reset_nasm (nasm_t *nasm);

/* ---- ready pool -------------------------------------------------------------------------- */
/* reference include/aspen.h:104-109.  input_data of rpool_add_nasm_raw_input is the dense input
   matrix (NHWC images, or [batch][seq][M] rows); it is copied, the caller keeps ownership.
   rpool_add_nasm reads an NCHW float file (NULL = zeros). */
rpool_t *rpool_init (void);
void rpool_destroy (rpool_t *rpool);
void rpool_add_nasm_raw_input (rpool_t *rpool, nasm_t *nasm, void *input_data);
void rpool_add_nasm (rpool_t *rpool, nasm_t *nasm, char *input_filename);
void rpool_reset_queue (rpool_t *rpool);
void rpool_reset_nasm (rpool_t *rpool, nasm_t *nasm);

/* ---- scheduling engines ------------------------------------------------------------------ */
/* reference include/aspen.h:111-120.  One dse_group drives one GPU: dse_group_run starts the
   device-side engine on every armed nasm of the group's rpool and returns at once;
   dse_wait_for_nasm_completion blocks until that nasm's last tile is done; dse_group_stop waits
   for the engine to drain.  Result buffers are malloc'd; the caller frees them. */
dse_group_t *dse_group_init (unsigned int num_dse);
void dse_group_set_rpool (dse_group_t *dse_group, rpool_t *rpool);
void dse_group_destroy (dse_group_t *dse_group);
void dse_group_run (dse_group_t *dse_group);
void dse_group_stop (dse_group_t *dse_group);
void dse_group_run_until_nasm_completion (dse_group_t *dse_group, nasm_t *nasm);
void dse_wait_for_nasm_completion (nasm_t *nasm);
unsigned int dse_check_nasm_completion (nasm_t *nasm);
ssize_t dse_get_ldata_result (nasm_t *nasm, unsigned int ldata_idx, LAYER_PARAMS *order, void **out_ptr);
ssize_t dse_get_nasm_result (nasm_t *nasm, LAYER_PARAMS *order, void **out_ptr);

/* reference include/aspen.h:122 */
void aspen_flush_dynamic_memory (void);

/* ---- dumps (reference include/aspen.h:124-133) -------------------------------------------- */
void print_aspen_build_info (void);
void print_dnn_info (aspen_dnn_t *dnn, int print_data);
void print_layer_info (aspen_layer_t *layer, int print_data);
void print_tensor_info (aspen_tensor_t *tensor, int print_data);
void print_nasm_info (nasm_t *nasm, int print_ninst, int print_data);
void print_ldata_info (nasm_ldata_t *ldata, int print_ninst, int print_data);
void print_ninst_info (ninst_t *ninst, int print_data);
void print_rpool_queue_info (rpool_queue_t *rpool_queue);
void print_rpool_queue_group_info (rpool_queue_group_t *rpool_queue_group);
void print_rpool_info (rpool_t *rpool);

#ifdef __cplusplus
}
#endif
#endif /* ASPEN_AMD_ASPEN_H */
