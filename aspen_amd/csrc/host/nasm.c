/*
 * nasm.c -- tile graph: per-layer matrices, GPU tile policy, analytic tile-to-tile dependencies.
 *
 * Counterpart of the reference's graph builder (reference src/apu_nasm.c):
 *   get_out_mat_info :950        -> matrix shape per layer (rows = channels, columns = batch x positions)
 *   get_ninst_tile_dims :1025,
 *   init_nasm_ldata :1062        -> tile policy; here sized for 256 compute units and the MFMA tile
 *                                   shapes instead of 64 x 12 CPU tiles
 *   ninst_find_parent :49-466    -> dependencies; the reference visits every output element times its
 *                                   receptive field, here each tile's parents follow from interval
 *                                   arithmetic on its column / row range
 *   apu_create_nasm :682, apu_create_transformer_nasm :715, apu_reset_nasm :753, apu_destroy_nasm :936
 */
#include "internal.h"

static unsigned int nasm_counter = 0;
#define WEIGHT_STREAM_BYTES (16u << 20)      /* see set_tiles */

static unsigned int cdiv (unsigned int a, unsigned int b) { return (a + b - 1) / b; }
static unsigned int umin (unsigned int a, unsigned int b) { return a < b ? a : b; }
static unsigned int umax (unsigned int a, unsigned int b) { return a > b ? a : b; }

/* column stride for a matrix with `rows` rows: 16-byte aligned columns, zero padded */
unsigned int aspen_ld_for_rows (unsigned int rows) { return cdiv (rows, 4) * 4; }

static int is_contraction (LAYER_TYPE t) { return t == CONV_LAYER || t == FC_LAYER || t == MATMUL_LAYER; }

/* matrix shape, flop count (reference src/apu_nasm.c:950-1023) */
static int set_out_mat (nasm_t *nasm, nasm_ldata_t *ld)
{
    const aspen_layer_t *L = ld->layer;
    const unsigned int *p = L->params;
    const unsigned int B = nasm->batch_size, S = nasm->tr_seq_len;
    uint64_t flop_per_out = 1;
    switch (L->type)
    {
    case CONV_LAYER:
        flop_per_out = 2ull * p[WEIGHT_H] * p[WEIGHT_W] * p[IN_C];
        ld->out_mat_dims[OUT_H] = p[OUT_C]; ld->out_mat_dims[OUT_W] = p[OUT_H] * p[OUT_W] * B;
        break;
    case FC_LAYER:
        flop_per_out = 2ull * p[IN_C] * p[IN_H] * p[IN_W];
        ld->out_mat_dims[OUT_H] = p[OUT_C]; ld->out_mat_dims[OUT_W] = B;
        break;
    case MAXPOOL_LAYER: case AVGPOOL_LAYER:
        flop_per_out = (uint64_t)p[WEIGHT_H] * p[WEIGHT_W];
        ld->out_mat_dims[OUT_H] = p[OUT_C]; ld->out_mat_dims[OUT_W] = p[OUT_H] * p[OUT_W] * B;
        break;
    case INPUT_LAYER: case RESIDUAL_LAYER: case YOLO_LAYER: case APPEND_LAYER:
        if (S != 0) { ld->out_mat_dims[OUT_H] = p[MAT_M]; ld->out_mat_dims[OUT_W] = S * B; }
        else { ld->out_mat_dims[OUT_H] = p[OUT_C]; ld->out_mat_dims[OUT_W] = p[OUT_H] * p[OUT_W] * B; }
        break;
    case SOFTMAX_LAYER:
        ld->out_mat_dims[OUT_H] = p[OUT_C]; ld->out_mat_dims[OUT_W] = B;
        break;
    case MATMUL_LAYER:
        flop_per_out = 2ull * p[MAT_K];
        ld->out_mat_dims[OUT_H] = p[MAT_M]; ld->out_mat_dims[OUT_W] = S * B;
        break;
    case K_ATTENTION_LAYER:
        if (p[NUM_HEAD] == 0) { ERROR_PRTF ("layer %u: attention layer without heads\n", L->layer_idx); return -1; }
        flop_per_out = 2ull * p[NUM_HIDDEN] / p[NUM_HEAD];
        ld->out_mat_dims[OUT_H] = S; ld->out_mat_dims[OUT_W] = S * p[NUM_HEAD] * B;
        break;
    case V_ATTENTION_LAYER:
        if (p[NUM_HEAD] == 0) { ERROR_PRTF ("layer %u: attention layer without heads\n", L->layer_idx); return -1; }
        flop_per_out = 2ull * S;
        ld->out_mat_dims[OUT_H] = p[MAT_M]; ld->out_mat_dims[OUT_W] = S * B;
        break;
    case LAYERNORM_LAYER:
        ld->out_mat_dims[OUT_H] = p[MAT_M]; ld->out_mat_dims[OUT_W] = S * B;
        break;
    default:
        ERROR_PRTF ("ERROR) Unsupported layer type %d\n", (int)L->type);
        return -1;
    }
    if (ld->out_mat_dims[OUT_H] == 0 || ld->out_mat_dims[OUT_W] == 0)
    {
        ERROR_PRTF ("layer %u has an empty output matrix (transformer graphs need a sequence length: use apu_create_transformer_nasm)\n", L->layer_idx);
        return -1;
    }
    ld->flops = flop_per_out * ld->out_mat_dims[OUT_H] * ld->out_mat_dims[OUT_W];
    /* the input keeps the tight 16-byte column alignment (3-channel images would otherwise be read
       8x); every matrix produced on the device gets 128-byte columns, so that no cache line is shared
       between two columns (and hence between two producer tiles), which lets consumers read it
       through the caches.  K-attention needs the multiple of 32 anyway: the V tile streams the
       probabilities 32 keys at a time. */
    ld->out_mat_stride = L->type == INPUT_LAYER ? aspen_ld_for_rows (ld->out_mat_dims[OUT_H]) : cdiv (ld->out_mat_dims[OUT_H], 32) * 32;
    return 0;
}

/* Tile policy.  min_ninst = wanted tiles per layer (the knob of apu_create_nasm): the largest tile
   shape that still yields that many tiles is taken, so big layers get the large MFMA tiles and
   small ones are cut finer to keep all compute units busy. */
static int set_tiles (nasm_t *nasm, nasm_ldata_t *ld)
{
    const aspen_layer_t *L = ld->layer;
    const unsigned int M = ld->out_mat_dims[OUT_H], N = ld->out_mat_dims[OUT_W];
    const unsigned int want = nasm->min_ninst_per_ldata;
    ld->variant = 0;
    ld->splits = 1; ld->kiters_per_split = 0;
    if (L->type == INPUT_LAYER)
    {
        ld->tile_dims[OUT_H] = M; ld->tile_dims[OUT_W] = N; ld->tiles_h = ld->tiles_w = 0; ld->num_ninst = 0;
        return 0;
    }
    if (is_contraction (L->type))
    {
        uint32_t shp[13];
        aspen_hip_tile_shapes (shp);
        const unsigned int bm[ASPEN_HIP_NUM_GEMM_VARIANTS] = {shp[0], shp[2], shp[4], shp[9], shp[11]}, bn[ASPEN_HIP_NUM_GEMM_VARIANTS] = {shp[1], shp[3], shp[5], shp[10], shp[12]};
        /* few output rows: the wide shape; otherwise the large one; either falls back to the small
           shape when it would leave the layer with fewer tiles than wanted */
        int v = M <= 64 ? ASPEN_HIP_GEMM_WIDE : ASPEN_HIP_GEMM_LARGE;
        if (cdiv (M, bm[v]) * cdiv (N, bn[v]) < want || (N <= 64 && v == ASPEN_HIP_GEMM_WIDE)) v = ASPEN_HIP_GEMM_SMALL;
        if (nasm->small_tiles_only) v = ASPEN_HIP_GEMM_SMALL;      /* graphs bound by their dependency chains, see create_nasm */
        if (nasm->kiters_cap && aspen_layer_kiters (L) > nasm->kiters_cap) v = ASPEN_HIP_GEMM_SMALL;   /* only the small shape is cut along K */
        if (aspen_layer_table_operand (L)) v = ASPEN_HIP_GEMM_SMALL;
        /* latency-bound graphs (see create_nasm): a layer that the 64 x 64 shape leaves with less than half the wanted tiles
           takes the 32 x 32 shape, whose four wavefronts split the K axis between them */
        if (nasm->narrow_tiles && v == ASPEN_HIP_GEMM_SMALL && !aspen_layer_table_operand (L) && !aspen_layer_dense3 (L)
            && 2 * cdiv (M, bm[v]) * cdiv (N, bn[v]) < want) v = ASPEN_HIP_GEMM_NARROW;
        /* A layer that streams a large weight matrix past at most 32 columns (the first FC layers of VGG-16 up to batch
           32: 411 MB and 67 MB of weights) takes the tall shape, 128 weight rows x 32 columns.  With 64 x 64 tiles half of
           every MFMA works on padding columns, and the layer is bound by the matrix pipeline at twice its useful work
           (411 MB in 116 us = 3.5 TB/s, whatever the number of tiles and whether or not the weights lie in memory in tile
           order -- both measured) instead of by the weights' trip from memory.  (The 32 x 32 shape, every wavefront
           reading its own rows and K range straight into registers, is slower still: 148 us; a lane pair per row and
           request makes poor use of the memory pipeline.  ASPEN_GPU_WEIGHT_STREAM=narrow / =off for comparisons.) */
        const char *wsb = getenv ("ASPEN_GPU_WEIGHT_STREAM_BYTES");       /* (tests: the shape on small layers) */
        if (N <= bn[ASPEN_HIP_GEMM_TALL] && (uint64_t)M * aspen_layer_kiters (L) * 32 * sizeof (float) >= (wsb ? strtoull (wsb, NULL, 10) : WEIGHT_STREAM_BYTES)
            && !aspen_layer_table_operand (L) && !aspen_layer_dense3 (L))
        {
            const char *e = getenv ("ASPEN_GPU_WEIGHT_STREAM");
            if (e == NULL || strcmp (e, "off") != 0) v = (e != NULL && strcmp (e, "narrow") == 0) ? ASPEN_HIP_GEMM_NARROW : ASPEN_HIP_GEMM_TALL;
        }
        ld->variant = v;
        ld->tile_dims[OUT_H] = bm[v]; ld->tile_dims[OUT_W] = bn[v];
        /* A short K axis (up to four slices) under the large shape: a tile is mostly set-up, first fetch and epilogue, so a
           workgroup takes two or four row tiles of its column block at a time while that still leaves the layer the tiles
           it wants (the 64 -> 256 channel layers of ResNet-50's first stage: 1568 tiles of 256 x 64 instead of 3136 of
           128 x 64). */
        if (v == ASPEN_HIP_GEMM_LARGE && aspen_layer_kiters (L) <= 4 && getenv ("ASPEN_GPU_NO_ROW_GROUPS") == NULL)
        {
            unsigned int r = 1;
            while (r < 4 && M >= bm[v] * 2 * r && cdiv (M, bm[v] * 2 * r) * cdiv (N, bn[v]) >= want) r *= 2;
            ld->tile_dims[OUT_H] = bm[v] * r;
        }
    }
    else if (L->type == K_ATTENTION_LAYER)
    {
        const unsigned int S = nasm->tr_seq_len, hd = L->params[NUM_HIDDEN] / L->params[NUM_HEAD];
        if (hd % 32 != 0) { ERROR_PRTF ("layer %u: head size %u must be a multiple of 32\n", L->layer_idx, hd); return -1; }
        uint32_t shp[13];
        aspen_hip_tile_shapes (shp);
        ld->tile_dims[OUT_H] = M; ld->tile_dims[OUT_W] = shp[6];
        ld->tiles_h = 1; ld->tiles_w = (N / S) * cdiv (S, shp[6]);
        ld->num_ninst = ld->tiles_w;
        return 0;
    }
    else if (L->type == V_ATTENTION_LAYER)
    {
        const unsigned int S = nasm->tr_seq_len, hd = L->params[NUM_HIDDEN] / L->params[NUM_HEAD];
        if (hd * L->params[NUM_HEAD] != M || (hd > 64 && hd % 64 != 0) || hd % 4 != 0)
        { ERROR_PRTF ("layer %u: unsupported head geometry (M %u, heads %u)\n", L->layer_idx, M, L->params[NUM_HEAD]); return -1; }
        uint32_t shp[13];
        aspen_hip_tile_shapes (shp);
        ld->tile_dims[OUT_H] = umin (hd, 64); ld->tile_dims[OUT_W] = shp[7];
        ld->tiles_h = M / ld->tile_dims[OUT_H]; ld->tiles_w = (N / S) * cdiv (S, shp[7]);
        ld->num_ninst = ld->tiles_h * ld->tiles_w;
        return 0;
    }
    else
    {
        /* bandwidth tiles: whole columns; start from 128 columns (the GEMM column tile, so edges
           line up) and halve until there are enough tiles */
        unsigned int tn = 128;
        if (L->type == SOFTMAX_LAYER || L->type == LAYERNORM_LAYER) tn = 32;
        while (tn > 4 && cdiv (N, tn) < want) tn /= 2;      /* small tiles finish sooner: measured better than fewer edges */
        while (tn < 1024 && (uint64_t)tn * ld->out_mat_stride < 16384 && cdiv (N, tn * 2) >= 2 * want) tn *= 2;
        ld->tile_dims[OUT_H] = M; ld->tile_dims[OUT_W] = tn;
        /* pooling layers with few output positions (global average pooling) are cut along the
           channels as well, in multiples of 32 rows */
        if ((L->type == MAXPOOL_LAYER || L->type == AVGPOOL_LAYER) && cdiv (N, tn) < want && M >= 64)
        {
            unsigned int tm = 256;
            while (tm > 32 && cdiv (N, tn) * cdiv (M, tm) < want) tm /= 2;
            if (tm < M) ld->tile_dims[OUT_H] = tm;
        }
    }
    ld->tiles_h = cdiv (M, ld->tile_dims[OUT_H]);
    ld->tiles_w = cdiv (N, ld->tile_dims[OUT_W]);
    ld->num_ninst = ld->tiles_h * ld->tiles_w;
    if (is_contraction (L->type))
    {
        /* still short of tiles with the smallest shape: cut the K axis (at least 8 slices of 32 per part) */
        const unsigned int kiters = aspen_layer_kiters (L), T = ld->num_ninst;
        ld->kiters_per_split = kiters;
        /* kiters_cap (graphs bound by their dependency chains, see create_nasm): no tile longer than that many K slices */
        const unsigned int cap = nasm->kiters_cap;
        if (ld->variant == ASPEN_HIP_GEMM_NARROW)
        {
            /* the workgroup's wavefronts already split K four ways: cut it across workgroups only while every wavefront
               keeps about three slices */
            const char *e1 = getenv ("ASPEN_GPU_NARROW_MAX_SPLITS"), *e2 = getenv ("ASPEN_GPU_NARROW_MIN_KITERS");
            const unsigned int max_splits = e1 ? (unsigned int)atoi (e1) : 16, min_kiters = e2 ? (unsigned int)atoi (e2) : 12;    /* (8 and 16 measured on ResNet-50 batch 1: 0.456 / 0.458 against 0.449 ms) */
            if (T < want && kiters >= 2 * min_kiters && getenv ("ASPEN_GPU_NO_SPLITK") == NULL)
            {
                unsigned int s = umin (umin (cdiv (want, T), kiters / umax (min_kiters, 1)), umax (max_splits, 1));
                ld->kiters_per_split = cdiv (kiters, umax (s, 1));
                ld->splits = cdiv (kiters, ld->kiters_per_split);
                if (ld->splits > 1) ld->num_ninst = T * ld->splits;
            }
        }
        else if ((T < want || (cap && kiters > cap)) && kiters >= 16 && getenv ("ASPEN_GPU_NO_SPLITK") == NULL)
        {
            /* (a tall tile's layer has few row tiles and a long K axis: up to 16 parts of at least 16 slices.  Measured on
               VGG-16 batch 32, each layer launched alone: 4096 x 25088 in 87 / 85 / 97 us with 8 / 16 / 32 parts, 4096 x 4096
               in 19.5 / 23.5 us with 8 / 16) */
            const int tall = ld->variant == ASPEN_HIP_GEMM_TALL;
            const char *e1 = getenv (tall ? "ASPEN_GPU_TALL_MAX_SPLITS" : "ASPEN_GPU_MAX_SPLITS"), *e2 = getenv (tall ? "ASPEN_GPU_TALL_MIN_KITERS" : "ASPEN_GPU_MIN_KITERS");
            const unsigned int max_splits = e1 ? (unsigned int)atoi (e1) : tall ? 16 : 8, min_kiters = e2 ? (unsigned int)atoi (e2) : tall ? 16 : 8;
            unsigned int s = umin (umin (umax (cdiv (want, T), cap ? cdiv (kiters, cap) : 1), kiters / umax (min_kiters, 1)), umax (max_splits, 1));
            ld->kiters_per_split = cdiv (kiters, s);
            ld->splits = cdiv (kiters, ld->kiters_per_split);
            if (ld->splits > 1) ld->num_ninst = T * ld->splits;
        }
    }
    return 0;
}

/* ---- tile geometry ---------------------------------------------------------------------------- */
/* Attention layers tile every sequence separately (a tile never crosses a (batch, head) block). */
static unsigned int seq_block (const nasm_ldata_t *ld)
{
    LAYER_TYPE t = ld->layer->type;
    return (t == K_ATTENTION_LAYER || t == V_ATTENTION_LAYER) ? ld->nasm->tr_seq_len : 0;
}

static unsigned int col_tile_of (const nasm_ldata_t *ld, unsigned int col)
{
    const unsigned int S = seq_block (ld), tw = ld->tile_dims[OUT_W];
    if (S == 0) return col / tw;
    return (col / S) * cdiv (S, tw) + (col % S) / tw;
}

static void tile_range (const nasm_ldata_t *ld, unsigned int t, unsigned int *c0, unsigned int *c1, unsigned int *r0, unsigned int *r1)
{
    if (ld->splits > 1) t /= ld->splits;
    const unsigned int tn = t / ld->tiles_h, tm = t % ld->tiles_h;      /* row tile fastest (reference src/apu_nasm.c:1218-1224) */
    const unsigned int S = seq_block (ld), tw = ld->tile_dims[OUT_W];
    if (S == 0) { *c0 = tn * tw; *c1 = umin (*c0 + tw, ld->out_mat_dims[OUT_W]); }
    else
    {
        const unsigned int per = cdiv (S, tw), blk = tn / per, q0 = (tn % per) * tw;
        *c0 = blk * S + q0; *c1 = blk * S + umin (q0 + tw, S);
    }
    *r0 = tm * ld->tile_dims[OUT_H]; *r1 = umin (*r0 + ld->tile_dims[OUT_H], ld->out_mat_dims[OUT_H]);
}

void aspen_nasm_tile_range_internal (const nasm_ldata_t *ld, unsigned int t, unsigned int *r)
{
    tile_range (ld, t, &r[0], &r[1], &r[2], &r[3]);
}

typedef struct { uint32_t *v; size_t n, cap; } u32vec;
static void push (u32vec *a, uint32_t x)
{
    if (a->n == a->cap)
    {
        const size_t cap = a->cap ? a->cap * 2 : 1024;
        uint32_t *v = realloc (a->v, cap * sizeof (uint32_t));
        if (v == NULL) { ERROR_PRTF ("ERROR: out of host memory while building the tile graph.\n"); abort (); }
        a->v = v; a->cap = cap;
    }
    a->v[a->n++] = x;
}

/* all tiles of `pl` that overlap columns [c0, c1) x rows [r0, r1) become parents */
static void add_parents (const nasm_ldata_t *pl, unsigned int c0, unsigned int c1, unsigned int r0, unsigned int r1, u32vec *out)
{
    if (pl->fused_into >= 0) pl = &pl->nasm->ldata_arr[pl->fused_into];   /* a fused shortcut is written by its contraction layer's tiles */
    if (pl->num_ninst == 0 || c1 <= c0 || r1 <= r0) return;   /* the input layer is complete from the start */
    c1 = umin (c1, pl->out_mat_dims[OUT_W]); r1 = umin (r1, pl->out_mat_dims[OUT_H]);
    const unsigned int t0 = col_tile_of (pl, c0), t1 = col_tile_of (pl, c1 - 1);
    const unsigned int m0 = r0 / pl->tile_dims[OUT_H], m1 = (r1 - 1) / pl->tile_dims[OUT_H];
    for (unsigned int t = t0; t <= t1; t++)
        for (unsigned int m = m0; m <= m1; m++)
            push (out, pl->ninst_start + (t * pl->tiles_h + m) * pl->splits);   /* split layer: slice 0 stands for the group */
}

/* parents of tile t of layer ld (semantics: reference src/apu_nasm.c:49-466) */
static void find_parents (const nasm_t *nasm, const nasm_ldata_t *ld, unsigned int t, u32vec *out)
{
    const aspen_layer_t *L = ld->layer;
    const unsigned int *p = L->params;
    const nasm_ldata_t *p0 = ld->parent_ldata_idx[PARENT_0] >= 0 ? &nasm->ldata_arr[ld->parent_ldata_idx[PARENT_0]] : NULL;
    const nasm_ldata_t *p1 = ld->parent_ldata_idx[PARENT_1] >= 0 ? &nasm->ldata_arr[ld->parent_ldata_idx[PARENT_1]] : NULL;
    unsigned int c0, c1, r0, r1;
    tile_range (ld, t, &c0, &c1, &r0, &r1);
    const unsigned int S = nasm->tr_seq_len;
    /* the tile that runs the epilogue of a layer with a fused shortcut also reads the shortcut's other
       operand; in a split layer that is whichever slice finishes last, so all of them wait for it */
    if (ld->fused_residual >= 0)
    {
        const nasm_ldata_t *res = &nasm->ldata_arr[ld->fused_residual];
        const nasm_ldata_t *other = &nasm->ldata_arr[res->parent_ldata_idx[PARENT_1]];
        if (other->stats_writer >= 0)
        {
            /* a folded norm: the epilogue normalises the norm's input itself, with the statistics the row-0 tiles of the
               norm's first folding layer have stored */
            add_parents (&nasm->ldata_arr[other->parent_ldata_idx[PARENT_0]], c0, c1, r0, r1, out);
            add_parents (&nasm->ldata_arr[other->stats_writer], c0, c1, 0, 1, out);
        }
        else add_parents (other, c0, c1, r0, r1, out);
    }
    /* A split-K partial tile of a pointwise layer (matmul, 1x1 convolution: the K index IS the parent's
       row index) reads only the parent rows of its K slice, so it waits only for the parent tiles
       holding those rows: fewer edges, and it can start before the rest of the parent is done. */
    unsigned int k_row0 = 0, k_row1 = p0 ? p0->out_mat_dims[OUT_H] : 0;
    if (ld->splits > 1
        && (L->type == MATMUL_LAYER || (L->type == CONV_LAYER && p[WEIGHT_H] == 1 && p[WEIGHT_W] == 1)))
    {
        const unsigned int slice = t % ld->splits;
        k_row0 = umin (slice * ld->kiters_per_split * 32, k_row1);
        k_row1 = umin ((slice + 1) * ld->kiters_per_split * 32, k_row1);
    }
    switch (L->type)
    {
    case CONV_LAYER: case MAXPOOL_LAYER: case AVGPOOL_LAYER:
    {
        const unsigned int ohw = p[OUT_H] * p[OUT_W], ihw = p[IN_H] * p[IN_W];
        const unsigned int pr0 = L->type == CONV_LAYER ? k_row0 : r0, pr1 = L->type == CONV_LAYER ? k_row1 : r1;
        for (unsigned int b = c0 / ohw; b <= (c1 - 1) / ohw; b++)
        {
            const unsigned int first = umax (c0, b * ohw) - b * ohw, last = umin (c1, (b + 1) * ohw) - 1 - b * ohw;
            const unsigned int oh0 = first / p[OUT_W], oh1 = last / p[OUT_W];
            int ih_lo = (int)(oh0 * p[STRIDE]) - (int)p[PADDING], ih_hi = (int)(oh1 * p[STRIDE]) - (int)p[PADDING] + (int)p[WEIGHT_H] - 1;
            int iw_lo = 0, iw_hi = (int)p[IN_W] - 1;
            if (oh0 == oh1)
            {
                iw_lo = (int)((first % p[OUT_W]) * p[STRIDE]) - (int)p[PADDING];
                iw_hi = (int)((last % p[OUT_W]) * p[STRIDE]) - (int)p[PADDING] + (int)p[WEIGHT_W] - 1;
            }
            if (ih_lo < 0) ih_lo = 0;
            if (iw_lo < 0) iw_lo = 0;
            if (ih_hi > (int)p[IN_H] - 1) ih_hi = (int)p[IN_H] - 1;
            if (iw_hi > (int)p[IN_W] - 1) iw_hi = (int)p[IN_W] - 1;
            if (ih_hi < ih_lo || iw_hi < iw_lo) continue;             /* window entirely in the padding */
            add_parents (p0, b * ihw + ih_lo * p[IN_W] + iw_lo, b * ihw + ih_hi * p[IN_W] + iw_hi + 1, pr0, pr1, out);
        }
        break;
    }
    case FC_LAYER:
    {
        const unsigned int ihw = p[IN_H] * p[IN_W];
        add_parents (p0, c0 * ihw, c1 * ihw, 0, p0->out_mat_dims[OUT_H], out);
        break;
    }
    case MATMUL_LAYER:
        /* (with a folded layer norm the tile reads the norm's input: whole columns, it gathers their statistics) */
        if (ld->folded_norm >= 0) p0 = &nasm->ldata_arr[nasm->ldata_arr[ld->folded_norm].parent_ldata_idx[PARENT_0]];
        add_parents (p0, c0, c1, k_row0, k_row1, out);
        break;
    case LAYERNORM_LAYER: case SOFTMAX_LAYER:
        add_parents (p0, c0, c1, 0, p0->out_mat_dims[OUT_H], out);
        break;
    case RESIDUAL_LAYER:
        add_parents (p0, c0, c1, r0, r1, out);
        add_parents (p1, c0, c1, r0, r1, out);
        break;
    case YOLO_LAYER:
    {
        /* output column = (batch, anchor, cell); it reads rows [anchor*R, anchor*R + R) of parent
           column (batch, cell) (reference src/tiled_kernels.c:686-697) */
        const unsigned int cells = p[IN_H] * p[IN_W], R = p[OUT_C], A = p[IN_C] / R;
        for (unsigned int c = c0; c < c1; )
        {
            const unsigned int seg = c / cells, b = seg / A, a = seg % A, cell0 = c % cells;
            const unsigned int end = umin (c1, (seg + 1) * cells), cell1 = cell0 + (end - c);
            add_parents (p0, b * cells + cell0, b * cells + cell1, a * R, (a + 1) * R, out);
            c = end;
        }
        break;
    }
    case APPEND_LAYER:
    {
        /* rows [0, IN_C): first parent, upsampled by `stride`; rows [IN_C, OUT_C): second parent at
           the output resolution (reference src/tiled_kernels.c:710-741) */
        const unsigned int ohw = p[OUT_H] * p[OUT_W], ihw = p[IN_H] * p[IN_W], st = p[STRIDE];
        add_parents (p1, c0, c1, 0, p1->out_mat_dims[OUT_H], out);
        for (unsigned int b = c0 / ohw; b <= (c1 - 1) / ohw; b++)
        {
            const unsigned int first = umax (c0, b * ohw) - b * ohw, last = umin (c1, (b + 1) * ohw) - 1 - b * ohw;
            const unsigned int ih0 = first / p[OUT_W] / st, ih1 = last / p[OUT_W] / st;
            unsigned int iw0 = 0, iw1 = p[IN_W] - 1;
            if (first / p[OUT_W] == last / p[OUT_W]) { iw0 = first % p[OUT_W] / st; iw1 = last % p[OUT_W] / st; }
            add_parents (p0, b * ihw + ih0 * p[IN_W] + iw0, b * ihw + ih1 * p[IN_W] + iw1 + 1, 0, p0->out_mat_dims[OUT_H], out);
        }
        break;
    }
    case K_ATTENTION_LAYER:
    {
        const unsigned int H = p[NUM_HEAD], hd = p[NUM_HIDDEN] / H;
        const unsigned int bh = c0 / S, b = bh / H, h = bh % H, q0 = c0 % S, q1 = q0 + (c1 - c0);
        add_parents (p0, b * S + q0, b * S + q1, h * hd, (h + 1) * hd, out);    /* Query columns of this tile */
        add_parents (p1, b * S, (b + 1) * S, h * hd, (h + 1) * hd, out);        /* every Key of the sequence */
        break;
    }
    case V_ATTENTION_LAYER:
    {
        const unsigned int H = p[NUM_HEAD], hd = p[NUM_HIDDEN] / H;
        const unsigned int b = c0 / S, h = r0 / hd, q0 = c0 % S, q1 = q0 + (c1 - c0);
        if (ld->fused_attention >= 0)
        {
            /* the tile computes its probabilities itself: it reads what the K-attention tile would have read */
            const nasm_ldata_t *kl = &nasm->ldata_arr[ld->fused_attention];
            add_parents (&nasm->ldata_arr[kl->parent_ldata_idx[PARENT_0]], b * S + q0, b * S + q1, h * hd, (h + 1) * hd, out);   /* its Queries */
            add_parents (&nasm->ldata_arr[kl->parent_ldata_idx[PARENT_1]], b * S, (b + 1) * S, h * hd, (h + 1) * hd, out);       /* every Key */
        }
        else add_parents (p0, (b * H + h) * S + q0, (b * H + h) * S + q1, 0, S, out); /* probability rows */
        add_parents (p1, b * S, (b + 1) * S, r0, r1, out);                       /* every Value of the sequence */
        break;
    }
    default: break;
    }
}

static int cmp_u32 (const void *a, const void *b)
{
    uint32_t x = *(const uint32_t *)a, y = *(const uint32_t *)b;
    return x < y ? -1 : x > y;
}

static int build_graph (nasm_t *nasm)
{
    const uint32_t n = nasm->num_ninst;
    nasm->ninst_ldata = calloc (n ? n : 1, sizeof (uint32_t));
    nasm->num_parents = calloc (n ? n : 1, sizeof (uint32_t));
    nasm->child_off = calloc ((size_t)n + 2, sizeof (uint32_t));
    u32vec edges_parent = {0}, edges_child = {0}, tmp = {0};
    if (nasm->ninst_ldata == NULL || nasm->num_parents == NULL || nasm->child_off == NULL) return -1;
    for (unsigned int l = 0; l < nasm->num_ldata; l++)
    {
        const nasm_ldata_t *ld = &nasm->ldata_arr[l];
        for (unsigned int t = 0; t < ld->num_ninst; t++)
        {
            const uint32_t id = ld->ninst_start + t;
            nasm->ninst_ldata[id] = l;
            tmp.n = 0;
            find_parents (nasm, ld, t, &tmp);
            qsort (tmp.v, tmp.n, sizeof (uint32_t), cmp_u32);
            uint32_t prev = 0xffffffffu;
            for (size_t i = 0; i < tmp.n; i++)
            {
                if (tmp.v[i] == prev) continue;         /* the two parents of a shortcut may be the same tile */
                prev = tmp.v[i];
                if (prev >= id)
                {
                    ERROR_PRTF ("tile %u depends on a later tile %u\n", id, prev);
                    free (edges_parent.v); free (edges_child.v); free (tmp.v);
                    return -1;
                }
                /* A parent in a split layer stands for its group of `splits` partial tiles: the member
                   that finishes last completes the output and releases the children, so every member
                   carries the child list and the child counts the group once. */
                const unsigned int members = nasm->ldata_arr[nasm->ninst_ldata[prev]].splits;
                for (unsigned int s = 0; s < members; s++)
                {
                    push (&edges_parent, prev + s); push (&edges_child, id);
                    nasm->child_off[prev + s + 1]++;
                }
                nasm->num_parents[id]++;
            }
        }
    }
    for (uint32_t i = 0; i < n; i++) nasm->child_off[i + 1] += nasm->child_off[i];
    nasm->num_edges = (uint32_t)edges_parent.n;
    nasm->child_idx = calloc (edges_parent.n ? edges_parent.n : 1, sizeof (uint32_t));
    uint32_t *cursor = calloc (n ? n : 1, sizeof (uint32_t));
    if (nasm->child_idx == NULL || cursor == NULL)
    {
        free (cursor); free (edges_parent.v); free (edges_child.v); free (tmp.v);
        return -1;
    }
    for (size_t e = 0; e < edges_parent.n; e++)
    {
        const uint32_t pnt = edges_parent.v[e];
        nasm->child_idx[nasm->child_off[pnt] + cursor[pnt]++] = edges_child.v[e];
    }
    free (cursor); free (edges_parent.v); free (edges_child.v); free (tmp.v);
    return 0;
}

/* Shortcut fusion.  out = act (p0 + p1) (reference tiled_residual, src/tiled_kernels.c:613-638) is a
   pure bandwidth layer and one more dependency level.  When p0 is a contraction layer that feeds only
   this shortcut, its tiles compute the shortcut in their epilogue: they still write p0's own matrix
   (every layer's output stays readable), read p1 at the same positions and write the shortcut's
   matrix too.  The shortcut layer keeps its matrix and loses its tiles. */
static void fuse_shortcuts (nasm_t *nasm)
{
    for (unsigned int r = 0; r < nasm->num_ldata; r++)
    {
        nasm_ldata_t *res = &nasm->ldata_arr[r];
        if (res->layer->type != RESIDUAL_LAYER) continue;
        const int i0 = res->parent_ldata_idx[PARENT_0], i1 = res->parent_ldata_idx[PARENT_1];
        if (i0 < 0 || i1 < 0 || i1 >= i0) continue;
        nasm_ldata_t *prod = &nasm->ldata_arr[i0];
        if (!is_contraction (prod->layer->type) || prod->fused_residual >= 0) continue;
        if (prod->out_mat_stride != res->out_mat_stride) continue;
        unsigned int consumers = 0;
        for (unsigned int l = 0; l < nasm->num_ldata; l++)
            for (int k = PARENT_0; k <= PARENT_1; k++)
                consumers += nasm->ldata_arr[l].parent_ldata_idx[k] == i0;
        if (consumers != 1) continue;
        prod->fused_residual = (int)r;
        res->fused_into = i0;
        /* nothing on the device reads the producer's own matrix any more; like the reference, which
           frees a layer's matrix once its children are done (src/dse.c:84-92), it is not kept unless asked */
        prod->out_discarded = !aspen_keep_layer_outputs_enabled ();
        res->num_ninst = 0; res->tiles_h = res->tiles_w = 0;
    }
}

/* Attention fusion.  The reference computes the S x S probabilities of every (batch, head) in one layer and
   multiplies them with the values in the next (tiled_k_attention / tiled_v_attention, src/tiled_kernels.c:784-1037),
   through memory.  When nothing else reads the probabilities and their matrix need not be kept, the V-attention
   layer's tiles compute both steps and the K-attention layer loses its tiles (its matrix is then not written, like
   the pre-shortcut matrix of a fused shortcut). */
static void fuse_attention (nasm_t *nasm)
{
    if (aspen_keep_layer_outputs_enabled () || getenv ("ASPEN_GPU_NO_FUSE_ATTENTION") != NULL) return;
    for (unsigned int v = 0; v < nasm->num_ldata; v++)
    {
        nasm_ldata_t *vl = &nasm->ldata_arr[v];
        if (vl->layer->type != V_ATTENTION_LAYER) continue;
        const int k = vl->parent_ldata_idx[PARENT_0];
        if (k < 0 || nasm->ldata_arr[k].layer->type != K_ATTENTION_LAYER) continue;
        nasm_ldata_t *kl = &nasm->ldata_arr[k];
        const unsigned int hd = vl->layer->params[NUM_HIDDEN] / vl->layer->params[NUM_HEAD];
        if (hd > 64 || hd % 32 != 0 || vl->tile_dims[OUT_H] != hd) continue;
        if (kl->layer->params[NUM_HEAD] != vl->layer->params[NUM_HEAD] || kl->layer->params[NUM_HIDDEN] != vl->layer->params[NUM_HIDDEN]) continue;
        unsigned int consumers = 0;
        for (unsigned int l = 0; l < nasm->num_ldata; l++)
            for (int p = PARENT_0; p <= PARENT_1; p++)
                consumers += nasm->ldata_arr[l].parent_ldata_idx[p] == k;
        if (consumers != 1 || kl->parent_ldata_idx[PARENT_0] < 0 || kl->parent_ldata_idx[PARENT_1] < 0) continue;
        vl->fused_attention = k;
        kl->out_discarded = 1;
        kl->num_ninst = 0; kl->tiles_h = kl->tiles_w = 0;
    }
}

/* Layer-norm folding.  y = W LN (x) + b is a product with the RAW column x, corrected afterwards with the column's mean
   and deviation (aspen_layer_norm_fold_to_device has the algebra).  A matmul layer in the 64 x 64 shape whose K axis is
   not cut reads every row of its columns in its K loop anyway and gathers the two sums on the way, so it need not wait
   for the norm's tiles.  A norm whose consumers can all do without its matrix is folded into them: it loses its tiles,
   its matrix is not written, and the graph is one dependency level shorter per norm.  Consumers that can:
   - such matmul layers (both norms of a pre-norm transformer block, GPT-2's: 4 x 512 tokens 3.70 -> 3.56 ms);
   - a shortcut that is computed in its producer's epilogue (the norms of a post-norm block, BERT's, are the
     shortcut's second operand): that epilogue normalises the norm's input itself, with the column statistics the
     row-0 tiles of the norm's first folding layer store (BERT-base 8 x 128 tokens: 2.07 -> 2.01 ms).  Folding only the
     matmul consumers and keeping the norm's tiles for the shortcut gains nothing (2.06 -> 2.07 ms: the tiles still
     have to run before the shortcut's reader).
   Not when layer outputs are kept. */
static void fold_layernorms (nasm_t *nasm)
{
    const char *e = getenv ("ASPEN_GPU_FOLD_LAYERNORM");
    if (aspen_keep_layer_outputs_enabled () || (e != NULL && atoi (e) == 0)) return;
    for (unsigned int n = 0; n + 1 < nasm->num_ldata; n++)        /* (the last layer's matrix is the result) */
    {
        nasm_ldata_t *nl = &nasm->ldata_arr[n];
        if (nl->layer->type != LAYERNORM_LAYER || nl->num_ninst == 0 || nl->parent_ldata_idx[PARENT_0] < 0) continue;
        const nasm_ldata_t *xl = &nasm->ldata_arr[nl->parent_ldata_idx[PARENT_0]];
        if (xl->out_mat_stride != nl->out_mat_stride || xl->out_mat_dims[OUT_H] != nl->out_mat_dims[OUT_H]) continue;
        unsigned int consumers = 0, able = 0, shortcuts = 0;
        int first_folding = -1;
        for (unsigned int l = 0; l < nasm->num_ldata; l++)
            for (int k = PARENT_0; k <= PARENT_1; k++)
            {
                const nasm_ldata_t *cl = &nasm->ldata_arr[l];
                if (cl->parent_ldata_idx[k] != (int)n) continue;
                consumers++;
                if (k == PARENT_0 && cl->layer->type == MATMUL_LAYER && cl->variant == ASPEN_HIP_GEMM_SMALL && cl->splits <= 1 && cl->num_ninst > 0
                    && cl->layer->gemm_k == nl->out_mat_dims[OUT_H] && cl->layer->gemm_k % 32 == 0)
                {
                    able++;
                    if (first_folding < 0) first_folding = (int)l;
                }
                /* a shortcut computed in its producer's epilogue (64 x 64 tiles over whole groups of 64 channels) can
                   normalise the norm's input there, given the column statistics: see aspen_hip_layer_t.fuse_norm_stats */
                else if (k == PARENT_1 && cl->layer->type == RESIDUAL_LAYER && cl->fused_into >= 0 && first_folding >= 0 && cl->fused_into > first_folding
                    && nasm->ldata_arr[cl->fused_into].variant == ASPEN_HIP_GEMM_SMALL && cl->out_mat_dims[OUT_H] % 64 == 0
                    && getenv ("ASPEN_GPU_NO_FOLD_SHORTCUT_NORM") == NULL)
                    shortcuts++;
            }
        if (able == 0 || consumers != able + shortcuts) continue;
        for (unsigned int l = 0; l < nasm->num_ldata; l++)
            if (nasm->ldata_arr[l].parent_ldata_idx[PARENT_0] == (int)n) nasm->ldata_arr[l].folded_norm = (int)n;
        if (shortcuts) nl->stats_writer = first_folding;
        nl->out_discarded = 1;
        nl->num_ninst = 0; nl->tiles_h = nl->tiles_w = 0;
    }
}

static nasm_t *build_nasm (aspen_dnn_t *dnn, unsigned int min_ninst, unsigned int batch, unsigned int seq, unsigned int kiters_cap, int small_tiles_only, int narrow_tiles)
{
    if (dnn == NULL) { ERROR_PRTF ("apu_create_nasm: dnn is NULL\n"); return NULL; }
    if (min_ninst < 1) { ERROR_PRTF ("ERROR: min_ninst_per_ldata should be at least 1\n"); return NULL; }
    nasm_t *nasm = calloc (1, sizeof (nasm_t));
    if (nasm == NULL) { ERROR_PRTF ("apu_create_nasm: out of host memory\n"); return NULL; }
    nasm->kiters_cap = kiters_cap;
    nasm->small_tiles_only = small_tiles_only;
    nasm->narrow_tiles = narrow_tiles;
    nasm->preferred_mode = -1;
    nasm->ordered_pref = -1;
    nasm->dnn = dnn; nasm->nasm_id = nasm_counter++;
    nasm->batch_size = batch > 0 ? batch : 1;
    nasm->tr_seq_len = seq; nasm->min_ninst_per_ldata = min_ninst;
    nasm->num_ldata = dnn->num_layers;
    nasm->ldata_arr = calloc (nasm->num_ldata ? nasm->num_ldata : 1, sizeof (nasm_ldata_t));
    if (nasm->ldata_arr == NULL) { ERROR_PRTF ("apu_create_nasm: out of host memory\n"); free (nasm); return NULL; }
    size_t arena = 0;
    unsigned int total = 0;
    int bad = 0;
    for (unsigned int l = 0; l < nasm->num_ldata && !bad; l++)
    {
        nasm_ldata_t *ld = &nasm->ldata_arr[l];
        ld->nasm = nasm; ld->layer = &dnn->layers[l];
        ld->fused_residual = ld->fused_into = ld->fused_attention = ld->folded_norm = ld->stats_writer = -1;
        ld->out_discarded = 0;
        for (int k = 0; k < NUM_PARENT_ELEMENTS; k++) ld->parent_ldata_idx[k] = ld->layer->parent_idx[k];
        if (set_out_mat (nasm, ld) || set_tiles (nasm, ld)) { bad = 1; break; }
        for (int k = PARENT_0; k <= PARENT_1; k++)
        {
            if (ld->parent_ldata_idx[k] < 0) continue;
            const nasm_ldata_t *pl = &nasm->ldata_arr[ld->parent_ldata_idx[k]];
            /* shortcut parents must have this layer's shape (reference src/tiled_kernels.c:613-638 reads both at the same (h, w)) */
            if (ld->layer->type == RESIDUAL_LAYER && (pl->out_mat_dims[OUT_H] != ld->out_mat_dims[OUT_H] || pl->out_mat_dims[OUT_W] != ld->out_mat_dims[OUT_W]))
            { ERROR_PRTF ("layer %u: shortcut parents differ in shape\n", l); bad = 1; }
        }
    }
    if (!bad && getenv ("ASPEN_GPU_NO_FUSE") == NULL) fuse_shortcuts (nasm);
    if (!bad) fuse_attention (nasm);
    if (!bad) fold_layernorms (nasm);
    for (unsigned int l = 0; l < nasm->num_ldata && !bad; l++)
    {
        nasm_ldata_t *ld = &nasm->ldata_arr[l];
        ld->out_mat_offset = arena;
        arena += ((size_t)ld->out_mat_stride * ld->out_mat_dims[OUT_W] + 63) / 64 * 64;    /* 256-byte aligned matrices */
        if (ld->splits > 1)
        {
            ld->partial_offset = arena;
            /* one block of tile_m x tile_n sums per slice and output tile (edge tiles included whole) */
            arena += (size_t)ld->splits * ld->tiles_h * ld->tiles_w * ld->tile_dims[OUT_H] * ld->tile_dims[OUT_W];
        }
        if (ld->stats_writer >= 0)
        {
            ld->stats_offset = arena;
            arena += ((size_t)2 * ld->out_mat_dims[OUT_W] + 63) / 64 * 64;
        }
        nasm->total_flops += ld->flops;
    }
    for (unsigned int l = 0; l < nasm->num_ldata && !bad; l++)
    {
        nasm_ldata_t *ld = &nasm->ldata_arr[l];
        ld->ninst_start = total;
        total += ld->num_ninst;
    }
    nasm->arena_floats = arena;
    nasm->num_ninst = total;
    if (!bad && build_graph (nasm)) bad = 1;
    if (bad) { dnn->ref_nasms++; apu_destroy_nasm (nasm); return NULL; }
    dnn->ref_nasms++;
    return nasm;
}

/* Average parallelism of a tile graph: summed tile cost over the cost of the longest dependency chain
   (cost = K slices of a contraction tile + a constant; the device library sizes its grid with the same
   estimate). */
static double nasm_parallelism (const nasm_t *nasm)
{
    const uint32_t n = nasm->num_ninst;
    if (n == 0) return 0.0;
    float *dist = calloc (n, sizeof (float));
    if (dist == NULL) return 0.0;
    double total = 0.0, longest = 0.0;
    for (uint32_t t = 0; t < n; t++)
    {
        const nasm_ldata_t *ld = &nasm->ldata_arr[nasm->ninst_ldata[t]];
        const LAYER_TYPE ty = ld->layer->type;
        float cost = 4.f;
        if (is_contraction (ty)) cost = 8.f + (ld->variant == ASPEN_HIP_GEMM_NARROW ? 0.25f : 1.f) * (float)(ld->splits > 1 ? ld->kiters_per_split : aspen_layer_kiters (ld->layer));
        else if (ty == K_ATTENTION_LAYER || ty == V_ATTENTION_LAYER) cost = 16.f;
        dist[t] += cost;
        total += cost;
        if (dist[t] > longest) longest = dist[t];
        for (uint32_t e = nasm->child_off[t]; e < nasm->child_off[t + 1]; e++)
            if (dist[nasm->child_idx[e]] < dist[t]) dist[nasm->child_idx[e]] = dist[t];      /* children have larger indices */
    }
    free (dist);
    return longest > 0.0 ? total / longest : 0.0;
}

/* A graph that offers less parallelism than a 256-CU device has resident workgroups is bound by its
   dependency chains, not by throughput: it runs on one or two workgroups per compute unit, and those idle while
   the longest tiles of each stage finish (BERT / GPT-2 with one or two thousand tokens).  Such a graph is rebuilt
   - with the small tile shape for every contraction layer: more and shorter tiles fill the rounds of a small grid
     better than few long ones (the FFN layers of BERT as 768 tiles instead of 384: GPT-2 -2 %, BERT -0.5 %);
   - if it still offers work for a second workgroup per compute unit, with no tile longer than 48 K slices (more
     split-K): GPT-2 (average parallelism 529) -6 %.  With a single workgroup per compute unit the extra tiles only
     queue up behind the others: BERT (265) is 2 % faster without the cap on the ready queue (in the ordered mode, which
     such transformer graphs now run, a cap of 24 pays: see create_nasm).
   Throughput-bound graphs (batch-32 vision nets) lose 2-3 % with either and keep their large, long tiles. */
#define CHAIN_BOUND_BELOW 1024.0
#define CHAIN_BOUND_CAP_FROM 400.0
#define CHAIN_BOUND_KITERS_CAP 48
#define ORDERED_KITERS_CAP 24
#define LATENCY_BOUND_BELOW 128.0
#define ORDERED_VISION_BELOW 1250.0
static nasm_t *create_nasm (aspen_dnn_t *dnn, unsigned int min_ninst, unsigned int batch, unsigned int seq)
{
    const char *e = getenv ("ASPEN_GPU_MAX_KITERS");            /* experiments: fixed cap, 0 = none */
    if (e != NULL) return build_nasm (dnn, min_ninst, batch, seq, (unsigned int)atoi (e), getenv ("ASPEN_GPU_SMALL_TILES") != NULL, getenv ("ASPEN_GPU_NARROW_TILES") != NULL);
    nasm_t *nasm = build_nasm (dnn, min_ninst, batch, seq, 0, 0, 0);
    if (nasm == NULL) return nasm;
    const double parallelism = nasm_parallelism (nasm);
    if (getenv ("ASPEN_GPU_VERBOSE")) fprintf (stderr, "aspen: graph of %u tiles, average parallelism %.0f\n", nasm->num_ninst, parallelism);
    if (parallelism >= CHAIN_BOUND_BELOW)
    {
        /* (convolutional graphs a little above the limit keep their tiles but still run better in the ordered mode,
           ordered / queue in ms: ResNet-50 batch 16, 1162: 1.49 / 1.53; VGG-16 batch 2 / 4 / 16 at 1052 / 1220 / 1234:
           0.80 / 0.91, 1.25 / 1.30, 3.94 / 4.09; from YOLO-v3 batch 8, 1271, on the queue wins: 4.76 / 4.68) */
        if (seq == 0 && parallelism < ORDERED_VISION_BELOW) nasm->ordered_pref = 1;
        return nasm;
    }
    /* bound by the LATENCY of its chains (one image through a deep network; the engine runs such a graph in its ordered
       mode): layers short of tiles take the 32 x 32 shape */
    const char *nt = getenv ("ASPEN_GPU_NARROW_TILES");
    const int narrow = nt != NULL ? atoi (nt) != 0 : parallelism < LATENCY_BOUND_BELOW;
    /* transformer graphs below the cap's limit run the ordered mode (below), where shorter tiles do pay: no tile longer
       than 24 K slices, i.e. the second FFN layer of a BERT-base block in four parts */
    const int tr_ordered = seq > 0 && parallelism < CHAIN_BOUND_CAP_FROM;
    nasm_t *rebuilt = build_nasm (dnn, min_ninst, batch, seq, parallelism >= CHAIN_BOUND_CAP_FROM ? CHAIN_BOUND_KITERS_CAP : tr_ordered ? ORDERED_KITERS_CAP : 0, 1, narrow);
    if (rebuilt == NULL) return nasm;
    /* The ordered mode itself pays further up than the 32 x 32 tiles do, for convolutional networks.  Measured against the
       ready queue (ms, ordered / queue): ResNet-50 at batch 1 / 2 / 4 / 8 / 16 (parallelism 95 / 175 / 335 / 593 / 790):
       0.45 / 0.64, 0.62 / 0.74, 0.72 / 0.88, 0.99 / 1.08, 1.47 / 1.62; YOLO-v3 at batch 1 / 2 / 4 (409 / 691 / 942): 1.24 / 1.57,
       1.71 / 1.94, 2.69 / 2.82; VGG-16 at batch 1 / 2 / 4 / 8 (583 / 654 / 766 / 884): 0.54 / 0.64, 0.82 / 0.85, 1.24 / 1.31,
       2.16 / 2.24.  Graphs that are not rebuilt here (1024 and up) are a tie or lose (YOLO-v3 batch 8, 1271: 4.76 / 4.68;
       ResNet-50 batch 32: 2.56 / 2.39).  Transformer graphs win with it below 400, together with the cap of 24 K slices
       (BERT-base, batch x tokens 8 x 128 / 4 x 128 / 8 x 64 / 2 x 384: 2.00 / 2.15, 1.38 / 1.46, 1.34 / 1.39, 1.90 / 2.08;
       GPT-2 1 x 512 / 2 x 256 / 8 x 128: 1.59 / 1.65, 1.43 / 1.50, 2.01 / 2.10); above, the times are within a percent or two
       of each other either way (GPT-2 4 x 512, 529: 3.56 / 3.60 on one box, 3.57 / 3.52 on another; BERT-base 16 x 128:
       3.34 / 3.38), and the ordered mode moves far less data: a tile's workgroup, and with it the XCD whose L2 its operands
       pass through, is fixed by the tile's index, so every XCD keeps to an eighth of a layer's weight rows.  So every
       rebuilt graph asks for the ordered mode.  Where it matters, apu_generate_nasm times both. */
    rebuilt->ordered_pref = 1;
    apu_destroy_nasm (nasm);
    return rebuilt;
}

nasm_t *apu_create_nasm (aspen_dnn_t *dnn, unsigned int min_ninst_per_ldata, unsigned int batch_size)
{
    return create_nasm (dnn, min_ninst_per_ldata, batch_size, 0);
}

nasm_t *apu_create_transformer_nasm (aspen_dnn_t *dnn, unsigned int min_ninst_per_ldata, unsigned int batch_size, unsigned int seq_num)
{
    return create_nasm (dnn, min_ninst_per_ldata, batch_size, seq_num);
}

/* ---- auto-tuner --------------------------------------------------------------------------------
   The reference searches the tile count by timing 50-iteration runs of candidate graphs on its DSE
   threads (reference src/apu_nasm.c:578-679: test_nasm_time_sec, apu_generate_nasm).  Same idea on the
   GPU: candidate values of min_ninst_per_ldata are built and timed on the dataflow engine (zero input,
   2 warm-up + 10 timed inferences each), the fastest wins.  num_iter = how many candidates beyond the
   default are tried, in the order below (nearest to the default first); 0 = take the default without
   timing.  Without a GPU the default is returned as well. */
#define DEFAULT_MIN_NINST 1536
#include <time.h>
/* large batches of vision nets like 1024-2048; transformers with a few hundred columns and batch 1 like
   few, large tiles (128-384) on one workgroup per compute unit */
static const unsigned int tuner_candidates[] = {DEFAULT_MIN_NINST, 384, 128, 768, 192, 1024, 2048, 256, 512, 3072};

static double test_nasm_time_sec (nasm_t *nasm, unsigned int iters, int mode)
{
    rpool_t *rpool = rpool_init ();
    dse_group_t *dse = dse_group_init (1);
    dse->mode = mode;
    dse_group_set_rpool (dse, rpool);
    rpool_add_nasm (rpool, nasm, NULL);
    struct timespec t0, t1;
    double sec = -1.0;
    int ok = 1;
    for (unsigned int i = 0; i < 2 + iters; i++)
    {
        if (i == 2) { aspen_hip_sync (); clock_gettime (CLOCK_MONOTONIC, &t0); }
        dse_group_run (dse);
        dse_wait_for_nasm_completion (nasm);
        dse_group_stop (dse);
        if (nasm->completed != 1) ok = 0;         /* a run the device gave up is no timing */
        rpool_reset_queue (rpool);
        rpool_reset_nasm (rpool, nasm);
    }
    if (aspen_hip_sync () == 0 && ok)
    {
        clock_gettime (CLOCK_MONOTONIC, &t1);
        sec = ((double)(t1.tv_sec - t0.tv_sec) + 1e-9 * (double)(t1.tv_nsec - t0.tv_nsec)) / (double)iters;
    }
    dse_group_destroy (dse);
    rpool_destroy (rpool);
    return sec;
}

static nasm_t *generate_nasm (aspen_dnn_t *dnn, unsigned int batch, unsigned int seq, unsigned int num_iter)
{
    const unsigned int ncand = sizeof (tuner_candidates) / sizeof (tuner_candidates[0]);
    if (num_iter == 0 || aspen_hip_init () != 0) return create_nasm (dnn, DEFAULT_MIN_NINST, batch, seq);
    static const char *const engine_name[3] = {"one launch per layer", "persistent kernel, ready queue", "persistent kernel, ordered"};
    unsigned int best = DEFAULT_MIN_NINST;
    int best_engine = 1;
    double best_time = -1.0;
    /* every candidate on the three engines: the persistent kernel with its ready queue (1) and in its ordered mode (2), one
       launch per layer (0) */
    for (unsigned int c = 0; c < ncand && c <= num_iter; c++)
    {
        nasm_t *cand = create_nasm (dnn, tuner_candidates[c], batch, seq);
        if (cand == NULL) return NULL;
        for (int engine = 2; engine >= 0; engine--)
        {
            cand->ordered_pref = engine == 2;
            const double t = test_nasm_time_sec (cand, 10, engine != 0);
            printf ("APU: min_ninst_per_ldata %u, %s: %u tiles, %f sec per inference\n", tuner_candidates[c], engine_name[engine], cand->num_ninst, t);
            fflush (stdout);
            if (t > 0 && (best_time < 0 || t < best_time)) { best_time = t; best = tuner_candidates[c]; best_engine = engine; }
        }
        apu_destroy_nasm (cand);
    }
    printf ("APU: NASM with min_ninst_per_ldata %u, %s, time = %f sec selected.\n", best, engine_name[best_engine], best_time);
    fflush (stdout);
    nasm_t *nasm = create_nasm (dnn, best, batch, seq);
    if (nasm != NULL)
    {
        nasm->preferred_mode = best_engine != 0;        /* what an engine group in mode "auto" will run it with */
        nasm->ordered_pref = best_engine == 2;
    }
    return nasm;
}

nasm_t *apu_generate_nasm (aspen_dnn_t *dnn, unsigned int batch_size, unsigned int num_iter)
{
    return generate_nasm (dnn, batch_size, 0, num_iter);
}
nasm_t *apu_generate_transformer_nasm (aspen_dnn_t *dnn, unsigned int batch_size, unsigned int seq_num, unsigned int num_iter)
{
    return generate_nasm (dnn, batch_size, seq_num, num_iter);
}

void apu_destroy_nasm (nasm_t *nasm)
{
    if (nasm == NULL) return;
    if (nasm->rpool != NULL)
    {
        rpool_t *rp = nasm->rpool;
        for (unsigned int i = 0; i < rp->num_nasms; i++)
            if (rp->nasms[i] == nasm)
            {
                memmove (&rp->nasms[i], &rp->nasms[i + 1], (rp->num_nasms - i - 1) * sizeof (nasm_t *));
                rp->num_nasms--;
                rp->graph_dirty = 1;
                break;
            }
    }
    if (nasm->d_arena != NULL) aspen_hip_sync ();      /* a run still in flight reads and writes the arena */
    aspen_hip_free (nasm->d_arena);
    free (nasm->ninst_ldata); free (nasm->num_parents); free (nasm->child_off); free (nasm->child_idx);
    free (nasm->ldata_arr);
    nasm->dnn->ref_nasms--;
    free (nasm);
}

void apu_reset_nasm (nasm_t *nasm)
{
    if (nasm == NULL) return;
    nasm->completed = 0;
    nasm->armed = 1;
}

/* ---- device ------------------------------------------------------------------------------------ */
int aspen_nasm_to_device (nasm_t *nasm)
{
    if (nasm->d_arena == NULL)
    {
        nasm->d_arena = aspen_hip_alloc (nasm->arena_floats * sizeof (float));
        if (nasm->d_arena == NULL) return -1;
    }
    for (unsigned int l = 0; l < nasm->num_ldata; l++)
    {
        nasm_ldata_t *ld = &nasm->ldata_arr[l];
        if (ld->parent_ldata_idx[PARENT_0] < 0) continue;
        if (aspen_layer_to_device (ld->layer, nasm->ldata_arr[ld->parent_ldata_idx[PARENT_0]].out_mat_stride)) return -1;
        if (ld->folded_norm >= 0 && aspen_layer_norm_fold_to_device (ld->layer, nasm->ldata_arr[ld->folded_norm].layer)) return -1;
    }
    return 0;
}

/* Device descriptors of all layers, tile indices shifted by ninst_base (position inside a merged graph);
   graph_id = which of the merged graphs this one is (the engine reports each one's completion separately). */
int aspen_nasm_fill_device_layers (nasm_t *nasm, aspen_hip_layer_t *dst, uint32_t ninst_base, uint32_t graph_id)
{
    for (unsigned int l = 0; l < nasm->num_ldata; l++)
    {
        const nasm_ldata_t *ld = &nasm->ldata_arr[l];
        const aspen_layer_t *L = ld->layer;
        const unsigned int *p = L->params;
        aspen_hip_layer_t *d = &dst[l];
        memset (d, 0, sizeof (*d));
        d->type = L->type; d->act = L->activation; d->variant = ld->variant;
        d->graph_id = graph_id;
        d->M = ld->out_mat_dims[OUT_H]; d->N = ld->out_mat_dims[OUT_W]; d->ld = ld->out_mat_stride;
        d->tile_m = ld->tile_dims[OUT_H]; d->tile_n = ld->tile_dims[OUT_W];
        d->tiles_m = ld->tiles_h; d->tiles_n = ld->tiles_w;
        d->ninst_start = ninst_base + ld->ninst_start; d->num_ninst = ld->num_ninst;
        d->splits = ld->splits; d->kiters_per_split = ld->kiters_per_split;
        d->partial = ld->splits > 1 ? nasm->d_arena + ld->partial_offset : NULL;
        d->out = nasm->d_arena + ld->out_mat_offset;
        if (ld->parent_ldata_idx[PARENT_0] >= 0)
        {
            const nasm_ldata_t *pl = &nasm->ldata_arr[ld->parent_ldata_idx[PARENT_0]];
            d->in0 = nasm->d_arena + pl->out_mat_offset; d->ld0 = pl->out_mat_stride;
        }
        if (ld->parent_ldata_idx[PARENT_1] >= 0)
        {
            const nasm_ldata_t *pl = &nasm->ldata_arr[ld->parent_ldata_idx[PARENT_1]];
            d->in1 = nasm->d_arena + pl->out_mat_offset; d->ld1 = pl->out_mat_stride;
        }
        d->weight = L->d_weight; d->bias = L->d_bias; d->ktab = L->d_ktab;
        d->K = L->gemm_k; d->Kp = L->dev_kp;
        d->IH = p[IN_H]; d->IW = p[IN_W]; d->IC = p[IN_C]; d->OH = p[OUT_H]; d->OW = p[OUT_W];
        d->KH = p[WEIGHT_H]; d->KW = p[WEIGHT_W]; d->stride = p[STRIDE]; d->pad = p[PADDING];
        if (L->type == FC_LAYER) { d->KH = p[IN_H]; d->KW = p[IN_W]; d->OH = 1; d->OW = 1; d->stride = 1; d->pad = 0; }
        if (L->type == MATMUL_LAYER) { d->IH = d->IW = d->OH = d->OW = d->KH = d->KW = d->stride = 1; d->pad = 0; d->IC = p[MAT_K]; }
        if (is_contraction (L->type))
        {
            const int pointwise = L->type == MATMUL_LAYER
                || (L->type == CONV_LAYER && p[WEIGHT_H] == 1 && p[WEIGHT_W] == 1 && p[STRIDE] == 1 && p[PADDING] == 0)
                || (L->type == FC_LAYER && p[IN_H] == 1 && p[IN_W] == 1);
            d->direct = pointwise && (d->IC % 32 == 0) && d->ld0 >= d->Kp;
            if (aspen_layer_dense3 (L)) d->direct = ASPEN_HIP_OPERAND_DENSE3;
        }
        if (ld->fused_residual >= 0)
        {
            const nasm_ldata_t *res = &nasm->ldata_arr[ld->fused_residual];
            const nasm_ldata_t *other = &nasm->ldata_arr[res->parent_ldata_idx[PARENT_1]];
            d->fuse_out = nasm->d_arena + res->out_mat_offset;
            d->fuse_in = nasm->d_arena + other->out_mat_offset; d->fuse_ld_in = other->out_mat_stride;
            if (other->stats_writer >= 0)
            {
                const nasm_ldata_t *xl = &nasm->ldata_arr[other->parent_ldata_idx[PARENT_0]];
                d->fuse_in = nasm->d_arena + xl->out_mat_offset; d->fuse_ld_in = xl->out_mat_stride;
                d->fuse_norm_stats = nasm->d_arena + other->stats_offset;
                d->fuse_norm_gamma = other->layer->d_weight; d->fuse_norm_beta = other->layer->d_bias;
            }
            d->fuse_act = res->layer->activation;
            d->fuse_discard = ld->out_discarded;
        }
        if (L->type == K_ATTENTION_LAYER || L->type == V_ATTENTION_LAYER)
        {
            d->heads = p[NUM_HEAD]; d->seq = nasm->tr_seq_len; d->hd = p[NUM_HIDDEN] / p[NUM_HEAD]; d->masked = p[MASKED];
        }
        if (ld->fused_attention >= 0)
        {
            /* in0 = Query, in1 = Key (the K-attention layer's parents), fuse_in = Value */
            const nasm_ldata_t *kl = &nasm->ldata_arr[ld->fused_attention];
            const nasm_ldata_t *ql = &nasm->ldata_arr[kl->parent_ldata_idx[PARENT_0]], *keyl = &nasm->ldata_arr[kl->parent_ldata_idx[PARENT_1]];
            const nasm_ldata_t *vl = &nasm->ldata_arr[ld->parent_ldata_idx[PARENT_1]];
            d->direct = ASPEN_HIP_ATTENTION_FUSED;
            d->in0 = nasm->d_arena + ql->out_mat_offset; d->ld0 = ql->out_mat_stride;
            d->in1 = nasm->d_arena + keyl->out_mat_offset; d->ld1 = keyl->out_mat_stride;
            d->fuse_in = nasm->d_arena + vl->out_mat_offset; d->fuse_ld_in = vl->out_mat_stride;
            d->masked = kl->layer->params[MASKED];
        }
        if (ld->folded_norm >= 0)
        {
            /* in0 = the norm's input; weights and bias with the norm's parameters folded in; in1 = the scaled weights' row sums */
            const nasm_ldata_t *nl = &nasm->ldata_arr[ld->folded_norm], *xl = &nasm->ldata_arr[nl->parent_ldata_idx[PARENT_0]];
            d->in0 = nasm->d_arena + xl->out_mat_offset; d->ld0 = xl->out_mat_stride;
            d->weight = L->d_weight_ln; d->bias = L->d_bias_ln; d->in1 = L->d_rowsum_ln; d->ld1 = 0;
            d->norm_fold = 1;
            if (nl->stats_writer == (int)l) d->norm_stats = nasm->d_arena + nl->stats_offset;
        }
    }
    return 0;
}
