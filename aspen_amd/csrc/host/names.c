/*
 * names.c -- printable names of the public enumerators, indexed by value
 * (reference include/aspen.h:67-73; the reference's tables are in src/util.c:3-41).
 * Every enumerator has a name here (the reference leaves COL_IDX_TENSOR and GELU_ACCURATE NULL).
 */
#include "aspen.h"

#define N(x) [x] = #x
char *ninst_state_str[NUM_NINST_STATES] = { N (NINST_NOT_READY), N (NINST_READY), N (NINST_COMPLETED) };
char *layer_type_str[NUM_LAYER_ELEMENTS] = {
    N (NO_LAYER_TYPE), N (INPUT_LAYER), N (CONV_LAYER), N (FC_LAYER), N (RESIDUAL_LAYER), N (BATCHNORM_LAYER), N (YOLO_LAYER),
    N (APPEND_LAYER), N (ACTIVATION_LAYER), N (MAXPOOL_LAYER), N (AVGPOOL_LAYER), N (ROUTE_LAYER), N (SOFTMAX_LAYER),
    N (MATMUL_LAYER), N (LAYERNORM_LAYER), N (K_ATTENTION_LAYER), N (V_ATTENTION_LAYER) };
char *param_type_str[NUM_PARAM_ELEMENTS] = {
    N (OUT_W), N (OUT_H), N (OUT_C), N (BATCH), N (IN_W), N (IN_H), N (IN_C), N (WEIGHT_W), N (WEIGHT_H), N (SUB_C), N (STRIDE),
    N (PADDING), N (DILATION), N (GROUPS), N (NUM_HIDDEN), N (NUM_HEAD), N (NUM_SEQ), N (MAT_M), N (MAT_N), N (MAT_K), N (SUB_M),
    N (MASKED), N (FORM_BYTES) };
char *tensor_type_str[NUM_TENSORS] = {
    N (NULL_TENSOR), N (OUTPUT_TENSOR), N (INPUT_TENSOR), N (WEIGHT_TENSOR), N (BIAS_TENSOR), N (COL_IDX_TENSOR), N (ANCHOR_TENSOR),
    N (BN_VAR_TENSOR), N (BN_MEAN_TENSOR), N (BN_WEIGHT_TENSOR) };
char *parent_type_str[NUM_PARENT_ELEMENTS] = { N (PARENT_NONE), N (PARENT_0), N (PARENT_1), N (PARENT_WEIGHT) };
char *activation_type_str[NUM_ACTIVATIONS] = {
    N (NO_ACTIVATION), N (SIGMOID), N (LINEAR), N (TANH), N (RELU), N (LEAKY_RELU), N (ELU), N (SELU), N (GELU), N (GELU_ACCURATE) };
char *rpool_cond_str[NUM_RPOOL_CONDS] = { N (RPOOL_DNN), N (RPOOL_LAYER_TYPE), N (RPOOL_LAYER_IDX), N (RPOOL_NASM), N (RPOOL_DSE) };
#undef N
