// Device-side tile arithmetic for gfx950 (MI355X): one function per tile class, each executed by one
// 256-thread workgroup (4 wavefronts of 64) on one output tile.  Shared by the per-layer launch
// kernel and the persistent dataflow kernel.
//
// Semantics follow the reference's per-ninst operators (reference src/tiled_kernels.c):
//   contraction tiles  tiled_conv2d :161, tiled_matmul :299, tiled_fully_connected :502
//                      (zero -> accumulate over K -> + bias -> activation)
//   tiled_residual :613, tiled_maxpool2d :411, tiled_avgpool2d :456, tiled_layernorm :743,
//   tiled_softmax :640, tiled_k_attention :784, tiled_v_attention :934
//   activation formulas: naive_activate, reference src/naive_kernels.c:11-57
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>
#include "aspen.h"
#include "aspen_hip.h"

typedef float floatx16 __attribute__ ((ext_vector_type (16)));

// Phase accounting of contraction tiles inside the persistent kernel (defined next to the kernel; costs one
// LDS read per call when profiling is off): 8 = operand set-up and first loads, 9 = K loop, 10 = epilogue,
// 11 = split-K arrival and reduction
__device__ void tile_phase_lap (int which);

#define WG_THREADS 256
#define GEMM_BK 32            // K floats staged per iteration: one 128-byte line per operand row
#define LDS_ROW 36            // floats per staged row: 32 + 4 padding -> conflict-free 128-bit reads

// Tiles of at most 128 x 64 outputs, 32 accumulator registers per lane, one LDS stage (the next K
// slice waits in registers) -> <= 128 VGPRs and <= 40 KB LDS per workgroup, so FOUR workgroups (16
// wavefronts) share a compute unit and one workgroup's load latency, epilogue and scheduling gaps are
// covered by the other three.  (128 x 128 tiles with two LDS stages and two workgroups per compute
// unit were measured too: better for very large GEMMs only, worse for every network here.)
#define VAR0_BM 128
#define VAR0_BN 64
#define WG_PER_CU 4
#define KATTN_BN 32            // queries per K-attention tile
#define VATTN_BN 64            // queries per V-attention tile
#define VAR1_BM 64
#define VAR1_BN 128
#define VAR2_BM 64
#define VAR2_BN 64
// The tall shape, for layers that stream a large weight matrix past a handful of columns (a fully connected layer at
// batch <= 32): four wavefronts, each 32 weight rows x the tile's 32 columns.  A 64 x 64 tile computes 32 columns of
// padding there, which makes such a layer bound by the matrix pipeline at twice its useful work instead of by the
// weights' trip from memory; this shape requests 16 KB of weights per K slice for the same number of MFMAs.
#define VAR4_BM 128
#define VAR4_BN 32
#define VAR4_DEPTH 2            // two slices of weights in flight: memory latency is all such a tile waits for
// K slices in flight from memory per tile shape (see gemm_core).  With two the larger shapes run out of registers
// (measured: ResNet-50 batch 32 2.81 -> 2.89 ms, VGG-16 7.90 -> 8.83 ms).  The small shape takes two for the matmul
// layers of transformer graphs, which run one or two workgroups per compute unit with nothing else to hide a slice's
// memory latency (BERT-base 2.45 -> 2.24 ms), and one in the kernels for convolutional networks: there four workgroups
// per compute unit hide it, and the second set of requests only lengthens the memory queues every tile's set-up
// waits in (YOLO-v3 batch 8 4.90 -> 4.84 ms, ResNet-50 batch 1 with one launch per layer 0.62 -> 0.60).
#define VAR0_DEPTH 1
#define VAR1_DEPTH 1
#define VAR2_DEPTH 2
#define SPLITK_TILE_FLOATS (VAR2_BM * VAR2_BN)     // one slice's sums of one output tile: a block of its own in `partial` (the tall shape has as many)
#define CMAX(a, b) ((a) > (b) ? (a) : (b))
#define STAGE_FLOATS(bm, bn) (((bm) + (bn)) * LDS_ROW)
#define EPI_FLOATS(bm, bn) ((bn) * ((bm) + 8))
#define VAR_FLOATS(bm, bn) CMAX (STAGE_FLOATS (bm, bn), EPI_FLOATS (bm, bn))
#define GEMM_SMEM_FLOATS CMAX (CMAX (VAR_FLOATS (VAR0_BM, VAR0_BN), VAR_FLOATS (VAR1_BM, VAR1_BN)), \
                               CMAX (VAR_FLOATS (VAR2_BM, VAR2_BN), STAGE_FLOATS (128, KATTN_BN)))
#define GEMM_SMEM_BYTES (GEMM_SMEM_FLOATS * 4)

// n / d for any 32-bit n, with {multiplier, shift} prepared on the host by divider_for (engine.hip):
// q = (((n - t) >> 1) + t) >> shift, t = high half of n * multiplier (the "round-up" method of division by an
// invariant integer, in its branch-free form, which is exact for every n and every d >= 2); bit 7 of shift marks d = 1.
__device__ __forceinline__ uint32_t fast_div (uint32_t n, const uint32_t (&dv)[2])
{
    const uint32_t t = __umulhi (n, dv[0]);
    const uint32_t q = (((n - t) >> 1) + t) >> (dv[1] & 31u);
    return (dv[1] & 0x80u) ? n : q;
}

__device__ __forceinline__ float4 ld4 (const float *p) { return *reinterpret_cast<const float4 *> (p); }
__device__ __forceinline__ void st4 (float *p, float4 v) { *reinterpret_cast<float4 *> (p) = v; }

// Loads from device memory through pointers the compiler cannot prove to be global (descriptor fields)
// would be FLAT instructions, which count as LDS traffic too: every wait for an LDS fragment would
// then also wait for them.  These go through the global address space explicitly.
typedef float floatx4 __attribute__ ((ext_vector_type (4)));
__device__ __forceinline__ float4 gld4 (const float *p)
{
    const floatx4 x = *(const floatx4 __attribute__ ((address_space (1))) *)p;
    return make_float4 (x[0], x[1], x[2], x[3]);
}
__device__ __forceinline__ float gld1 (const float *p) { return *(const float __attribute__ ((address_space (1))) *)p; }

// View of one activation matrix.  COH selects how it is accessed:
//   0  cached loads and write-back stores: the one-launch-per-layer path, where kernel boundaries provide
//      coherence.
//   1  every access is device-scope coherent (buffer instructions with sc1): loads bypass the per-CU
//      L1 and the per-XCD L2 (which are not coherent across the 8 XCDs), stores write through, so
//      tiles produced and consumed inside one persistent kernel need no cache write-back /
//      invalidate between them, and the weights stay cached.
//   2  stores write through (sc1), loads are cached.  Correct when no cache line of an activation is
//      shared by two producer tiles (the host checks strides and tile heights): a line is first
//      fetched after its only producer has finished, every element is written once per launch, and
//      the caches start a launch invalidated, so a cached line can never be stale.
// Offsets are in floats from the start of the matrix.  In modes 1 and 2 the buffer descriptor bounds-checks
// them in hardware (out-of-range loads return 0, out-of-range stores are dropped); mode 0 relies on the slack
// every allocation carries for the few floats an edge tile reads past a row.
typedef uint32_t u32x4 __attribute__ ((ext_vector_type (4)));
#define CPOL_SC1 16
template <int COH> struct ActView
{
    // COH != 0: buffer descriptor.  COH == 0: uniform base address for global loads / stores with 32-bit
    // offsets (measured: lower latency than buffer instructions, which counts when a single image runs
    // through one launch per layer; 64-bit pointers per row instead cost that kernel enough registers
    // to spill the weight pointers into the middle of its first loads).
    __amdgpu_buffer_rsrc_t rsrc;
    char __attribute__ ((address_space (1))) *base;
    static constexpr int LOAD_POLICY = COH == 1 ? CPOL_SC1 : 0, STORE_POLICY = COH ? CPOL_SC1 : 0;
    __device__ __forceinline__ void init (const float *p, uint32_t columns, uint32_t ld)
    {
        if (COH) rsrc = __builtin_amdgcn_make_buffer_rsrc ((void *)p, 0, (int)(columns * ld * 4u + 256u), 0x00020000);
        else base = (char __attribute__ ((address_space (1))) *)p;
    }
    __device__ __forceinline__ float4 ld4 (uint32_t off) const
    {
        if (COH) return __builtin_bit_cast (float4, __builtin_amdgcn_raw_buffer_load_b128 (rsrc, (int)(off * 4u), 0, LOAD_POLICY));
        const floatx4 x = *(const floatx4 __attribute__ ((address_space (1))) *)(base + off * 4u);
        return make_float4 (x[0], x[1], x[2], x[3]);
    }
    // ok ? ld4 (off) : zeros.  With a buffer descriptor the choice is made on the offset (one past anything the
    // descriptor covers reads as zeros): no branch around the load, so a K loop that uses it stays one basic block.
    __device__ __forceinline__ float4 ld4_if (uint32_t off, bool ok) const
    {
        if (COH) return __builtin_bit_cast (float4, __builtin_amdgcn_raw_buffer_load_b128 (rsrc, ok ? (int)(off * 4u) : (int)0xfffffff0u, 0, LOAD_POLICY));
        return ok ? ld4 (off) : make_float4 (0.f, 0.f, 0.f, 0.f);
    }
    __device__ __forceinline__ float ld1 (uint32_t off) const
    {
        if (COH) return __builtin_bit_cast (float, __builtin_amdgcn_raw_buffer_load_b32 (rsrc, (int)(off * 4u), 0, LOAD_POLICY));
        return *(const float __attribute__ ((address_space (1))) *)(base + off * 4u);
    }
    __device__ __forceinline__ void st4 (uint32_t off, float4 v) const
    {
        if (COH) __builtin_amdgcn_raw_buffer_store_b128 (__builtin_bit_cast (u32x4, v), rsrc, (int)(off * 4u), 0, STORE_POLICY);
        else *(floatx4 __attribute__ ((address_space (1))) *)(base + off * 4u) = (floatx4){v.x, v.y, v.z, v.w};
    }
    __device__ __forceinline__ void st1 (uint32_t off, float v) const
    {
        if (COH) __builtin_amdgcn_raw_buffer_store_b32 (__builtin_bit_cast (uint32_t, v), rsrc, (int)(off * 4u), 0, STORE_POLICY);
        else *(float __attribute__ ((address_space (1))) *)(base + off * 4u) = v;
    }
};

// The two GELU forms in single precision.  The reference's C expressions (src/naive_kernels.c:44-55)
// promote to double around a single-precision erff / tanhf; the results agree to about 1e-7 relative,
// three orders of magnitude inside the parity tolerance, and the transformer FFN epilogues spend a
// quarter of their time here.  tanh (u) = 1 - 2 / (exp (2u) + 1) with the hardware exponential:
// exp overflows to +inf for large u (-> 1) and underflows to 0 for very negative u (-> -1).
__device__ __forceinline__ float gelu_erf (float x) { return 0.5f * x * (1.f + erff (x * 0.7071067811865475f)); }
__device__ __forceinline__ float gelu_tanh (float x)
{
    const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
    const float t = 1.f - 2.f * __frcp_rn (__expf (2.f * u) + 1.f);
    return 0.5f * x * (1.f + t);
}

// Activations other than the three cheap ones.  The rare ones follow the reference's C expressions, which
// evaluate in double (reference src/naive_kernels.c:11-57).  Their code is large (erff, exp, double-precision
// constants), so they live in real functions: inlined into every epilogue copy they multiplied the
// kernel's code far beyond the instruction cache, and their constants were set up in front of the
// persistent loop and occupied registers during every tile.
__device__ __noinline__ float activate_slow (float x, int act)
{
    switch (act)
    {
    case ELU:           return x > 0 ? x : (float)(0.1 * (exp ((double)x) - 1));
    case SELU:          return x > 0 ? (float)(1.0507 * (double)x) : (float)(1.0507 * 1.67326 * (exp ((double)x) - 1));
    case SIGMOID:       return (float)(1 / (1 + exp (-(double)x)));
    case TANH:          return (float)tanh ((double)x);
    case GELU:          return gelu_erf (x);
    case GELU_ACCURATE: return gelu_tanh (x);
    default:            return x;
    }
}

// four values per call: the epilogues work on 16-byte pieces
__device__ __noinline__ float4 activate_slow4 (float4 v, int act)
{
    if (act == GELU) return make_float4 (gelu_erf (v.x), gelu_erf (v.y), gelu_erf (v.z), gelu_erf (v.w));
    if (act == GELU_ACCURATE) return make_float4 (gelu_tanh (v.x), gelu_tanh (v.y), gelu_tanh (v.z), gelu_tanh (v.w));
    return make_float4 (activate_slow (v.x, act), activate_slow (v.y, act), activate_slow (v.z, act), activate_slow (v.w, act));
}

__device__ __forceinline__ float activate (float x, int act)
{
    switch (act)
    {
    case NO_ACTIVATION: case LINEAR: return x;
    case RELU:          return x > 0 ? x : 0;
    case LEAKY_RELU:    return x > 0 ? x : (float)(0.1 * (double)x);
    default:            return activate_slow (x, act);
    }
}

__device__ __forceinline__ float4 act4 (float4 v, int act)
{
    switch (act)
    {
    case NO_ACTIVATION: case LINEAR: return v;
    case RELU:          return make_float4 (v.x > 0 ? v.x : 0, v.y > 0 ? v.y : 0, v.z > 0 ? v.z : 0, v.w > 0 ? v.w : 0);
    case LEAKY_RELU:    return make_float4 (activate (v.x, act), activate (v.y, act), activate (v.z, act), activate (v.w, act));
    default:            return activate_slow4 (v, act);
    }
}

// ---------------------------------------------------------------------------------------------
// Operand loaders.  A loader fetches this thread's share of one GEMM_BK-wide K slice into registers
// (load) and later parks it in LDS as [row][LDS_ROW] (store), so the global loads of slice i+1 fly
// while the matrix cores work on slice i.
// ---------------------------------------------------------------------------------------------

// Rows are K-contiguous in memory: weights [M][Kp], matmul / 1x1-conv activations, Q and K rows.
template <int ROWS> struct RowLoader
{
    static constexpr int R = ROWS / 32;
    // One uniform base pointer plus 32-bit byte offsets: global loads with a scalar base address need one
    // vector register per row instead of a 64-bit pointer.
    const char *base;
    uint32_t off[R], chunk, row0;
    // `rows` x `ld` floats at `p`, rows padded so that a tile never runs past them
    __device__ __forceinline__ void init (const float *p, uint32_t first_row, uint32_t rows, uint32_t ld, uint32_t tid)
    {
        (void)rows;
        chunk = tid & 7; row0 = tid >> 3;
        base = reinterpret_cast<const char *> (p);
        #pragma unroll
        for (int i = 0; i < R; i++) off[i] = ((first_row + row0 + 32u * i) * ld + chunk * 4u) * 4u;
    }
    __device__ __forceinline__ void load (int it, float4 (&v)[R])
    {
        #pragma unroll
        for (int i = 0; i < R; i++)
        {
            // the address space makes this a global (not flat) load whose 64-bit base stays in scalar registers
            typedef const floatx4 __attribute__ ((address_space (1))) global_floatx4;
            const char __attribute__ ((address_space (1))) *g = (const char __attribute__ ((address_space (1))) *)base;
            const floatx4 x = *(global_floatx4 *)(g + (off[i] + (uint32_t)it * (GEMM_BK * 4u)));
            v[i] = make_float4 (x[0], x[1], x[2], x[3]);
        }
    }
    __device__ __forceinline__ void store (float *lds, const float4 (&v)[R])
    {
        #pragma unroll
        for (int i = 0; i < R; i++) st4 (lds + (row0 + 32 * i) * LDS_ROW + chunk * 4, v[i]);
    }
};

// Same for rows of an activation matrix (matmul / 1x1-conv operand, Q, K and probability rows).
template <int ROWS, int COH> struct ActRowLoader
{
    static constexpr int R = ROWS / 32;
    ActView<COH> view;
    uint32_t off[R];
    uint32_t chunk, row0;
    // rows first_row.. of the view (clamped to max_row), starting at float `col0` of each row
    __device__ __forceinline__ void init (const ActView<COH> &v, uint32_t first_row, uint32_t max_row, uint32_t ld, uint32_t col0, uint32_t tid)
    {
        view = v; chunk = tid & 7; row0 = tid >> 3;
        #pragma unroll
        for (int i = 0; i < R; i++)
        {
            uint32_t r = first_row + row0 + 32 * i;
            r = r < max_row ? r : max_row;
            off[i] = r * ld + col0 + chunk * 4;
        }
    }
    __device__ __forceinline__ void load (int it, float4 (&v)[R])
    {
        #pragma unroll
        for (int i = 0; i < R; i++) v[i] = view.ld4 (off[i] + it * GEMM_BK);
    }
    __device__ __forceinline__ void store (float *lds, const float4 (&v)[R])
    {
        #pragma unroll
        for (int i = 0; i < R; i++) st4 (lds + (row0 + 32 * i) * LDS_ROW + chunk * 4, v[i]);
    }
};

// Implicit-GEMM activation operand of conv / FC: row n = output position (b, oh, ow); the K axis runs
// over (kh, kw, ic) and is resolved through the layer's k-chunk table.  Replaces the reference's
// pointer table + panel gather (prepare_input / load_im2col_ptr, reference src/tiled_kernels.c:3-159).
// TABLE: the K axis is resolved through the layer's k-chunk table (channel counts that are not multiples of the slice
// width, where a slice straddles taps; 64 x 64 tiles only, the host's tile policy sees to that).  Otherwise a whole
// slice belongs to one tap, found with a few scalar operations: fetching the table entry instead puts a dependent
// memory access in front of the operand loads of every slice.  Two loaders, not one with a branch: with both
// paths in one K loop the compiler waits for ALL outstanding loads wherever they join.
// K order of the stepping form (the host packs the weights to match): (channel block of 32, kh, kw, channel in block),
// i.e. consecutive slices walk the TAPS of one block of 32 channels.  The windows of neighbouring taps overlap, so a
// slice mostly re-reads what the previous one or the one KW before it fetched, while it is still in the caches; with
// the taps outermost (the reference's order) a tap's data came round again only after a whole pass over the channels,
// by which time a busy L2 had replaced it, and a 3 x 3 layer fetched its input up to nine times over the fabric.
template <int ROWS, int COH, bool TABLE> struct ConvLoader
{
    static constexpr int R = ROWS / 32;
    ActView<COH> in;
    const aspen_hip_ktab_t *ktab;
    int32_t base[R], ih0[R], iw0[R];
    uint32_t IH, IW, chunk, row0;
    uint32_t KH, KW, ld0;
    uint32_t kh, kw, c;                     // tap and channel the next slice asked for starts at (!TABLE)
    // first_it: the first K slice that will be asked for
    __device__ __forceinline__ void init (const aspen_hip_layer_t &L, const ActView<COH> &v, uint32_t first_row, uint32_t tid, int first_it)
    {
        in = v; IH = L.IH; IW = L.IW;
        chunk = tid & 7; row0 = tid >> 3;
        if (TABLE) ktab = L.ktab;
        else
        {
            KH = L.KH; KW = L.KW; ld0 = L.ld0;
            kh = kw = c = 0;
            if (first_it)
            {
                const uint32_t taps = KH * KW, block = (uint32_t)first_it / taps, tap = (uint32_t)first_it - block * taps;
                c = block * GEMM_BK;
                kh = tap / KW; kw = tap - kh * KW;
            }
        }
        const uint32_t ohw = L.OH * L.OW;
        #pragma unroll
        for (int i = 0; i < R; i++)
        {
            uint32_t n = first_row + row0 + 32 * i;
            n = n < L.N ? n : L.N - 1;
            uint32_t b = fast_div (n, L.div_ohw), rem = n - b * ohw, oh = fast_div (rem, L.div_ow), ow = rem - oh * L.OW;
            ih0[i] = (int32_t)(oh * L.stride) - (int32_t)L.pad;
            iw0[i] = (int32_t)(ow * L.stride) - (int32_t)L.pad;
            base[i] = ((int32_t)(b * L.IH) + ih0[i]) * (int32_t)L.IW * (int32_t)L.ld0 + iw0[i] * (int32_t)L.ld0;
        }
    }
    __device__ __forceinline__ void load (int it, float4 (&v)[R])
    {
        aspen_hip_ktab_t e;
        if (TABLE)
        {
            typedef unsigned int uintx2 __attribute__ ((ext_vector_type (2)));
            const uintx2 raw = *(const uintx2 __attribute__ ((address_space (1))) *)(ktab + it * 8 + chunk);
            e.offset = (int32_t)raw[0]; e.kh = (uint16_t)(raw[1] & 0xffffu); e.kw = (uint16_t)(raw[1] >> 16);
        }
        else
        {
            // Slices are asked for in ascending order from the one init was told, so the position is stepped, not
            // divided out, and `it` is not looked at.  (The K loops ask for the last slice once more than they need
            // and drop the answer: that request is one step past the K axis, i.e. the first tap again at the channels
            // behind the last block: the 128 bytes that follow the pixel's channel run, which exist for every pixel
            // but the matrix's last, where they lie in the slack behind the allocation.)
            e.offset = (int32_t)((kh * IW + kw) * ld0 + c + chunk * 4);
            e.kh = (uint16_t)kh; e.kw = (uint16_t)kw;
            if (++kw == KW) { kw = 0; if (++kh == KH) { kh = 0; c += GEMM_BK; } }
        }
        #pragma unroll
        for (int i = 0; i < R; i++)
        {
            const bool ok = (uint32_t)(ih0[i] + (int32_t)e.kh) < IH && (uint32_t)(iw0[i] + (int32_t)e.kw) < IW;
            v[i] = in.ld4_if ((uint32_t)(base[i] + e.offset), ok);
        }
    }
    __device__ __forceinline__ void store (float *lds, const float4 (&v)[R])
    {
        #pragma unroll
        for (int i = 0; i < R; i++) st4 (lds + (row0 + 32 * i) * LDS_ROW + chunk * 4, v[i]);
    }
};

// Implicit-GEMM operand of a convolution over THREE input channels (a network's first layer on RGB images) with a
// dense K axis: K order (tap, channel) without the padding to four channels per tap that ConvLoader's layout has
// (ASPEN_HIP_OPERAND_DENSE3; the stem of ResNet-50 contracts 160 instead of 224, VGG-16's first layer 32 instead of
// 64).  A chunk of four K positions spans two pixels: both are fetched (16 bytes each, the pixels of the matrix keep
// their padded fourth float) and the chunk is put together from the last channels of the first and the first
// channels of the second; chunk index % 3 says how many of each.  A loader of its own so that ConvLoader's code, which
// every other convolution runs, stays as it is.
template <int ROWS, int COH> struct Dense3Loader
{
    static constexpr int R = ROWS / 32;
    ActView<COH> in;
    const aspen_hip_ktab_t *ktab;
    int32_t base[R], ih0[R], iw0[R];
    uint32_t IH, IW, chunk, row0;
    __device__ __forceinline__ void init (const aspen_hip_layer_t &L, const ActView<COH> &v, uint32_t first_row, uint32_t tid)
    {
        in = v; ktab = L.ktab; IH = L.IH; IW = L.IW;
        chunk = tid & 7; row0 = tid >> 3;
        const uint32_t ohw = L.OH * L.OW;
        #pragma unroll
        for (int i = 0; i < R; i++)
        {
            uint32_t n = first_row + row0 + 32 * i;
            n = n < L.N ? n : L.N - 1;
            uint32_t b = fast_div (n, L.div_ohw), rem = n - b * ohw, oh = fast_div (rem, L.div_ow), ow = rem - oh * L.OW;
            ih0[i] = (int32_t)(oh * L.stride) - (int32_t)L.pad;
            iw0[i] = (int32_t)(ow * L.stride) - (int32_t)L.pad;
            base[i] = ((int32_t)(b * L.IH) + ih0[i]) * (int32_t)L.IW * (int32_t)L.ld0 + iw0[i] * (int32_t)L.ld0;
        }
    }
    __device__ __forceinline__ void load (int it, float4 (&v)[R])
    {
        typedef unsigned int uintx4 __attribute__ ((ext_vector_type (4)));
        const uint32_t kc = (uint32_t)it * 8 + chunk, sel = kc - 3 * ((kc * 43u) >> 7);        // kc % 3 for kc < 128
        const uintx4 raw = *(const uintx4 __attribute__ ((address_space (1))) *)(ktab + 2 * kc);
        #pragma unroll
        for (int i = 0; i < R; i++)
        {
            const bool oka = (uint32_t)(ih0[i] + (int32_t)(raw[1] & 0xffffu)) < IH && (uint32_t)(iw0[i] + (int32_t)(raw[1] >> 16)) < IW;
            const bool okb = (uint32_t)(ih0[i] + (int32_t)(raw[3] & 0xffffu)) < IH && (uint32_t)(iw0[i] + (int32_t)(raw[3] >> 16)) < IW;
            const float4 a = in.ld4_if ((uint32_t)(base[i] + (int32_t)raw[0]), oka), b = in.ld4_if ((uint32_t)(base[i] + (int32_t)raw[2]), okb);
            v[i].x = sel == 0 ? a.x : sel == 1 ? a.y : a.z;
            v[i].y = sel == 0 ? a.y : sel == 1 ? a.z : b.x;
            v[i].z = sel == 0 ? a.z : sel == 1 ? b.x : b.y;
            v[i].w = sel == 0 ? b.x : sel == 1 ? b.y : b.z;
        }
    }
    __device__ __forceinline__ void store (float *lds, const float4 (&v)[R])
    {
        #pragma unroll
        for (int i = 0; i < R; i++) st4 (lds + (row0 + 32 * i) * LDS_ROW + chunk * 4, v[i]);
    }
};

// K-strided operand (V of attention: rows = channels, K axis = sequence position with stride ld):
// read 64 channels x 32 positions with 128-bit loads along the channels, transpose into LDS.
template <int COH> struct TransLoader64
{
    static constexpr int R = 2;
    ActView<COH> view;
    uint32_t off[2];
    uint32_t c4, s0, ld, klen;
    bool live;
    // first: float offset of (position 0, first channel of the tile); valid_rows: channels of this tile
    // that exist; klen: length of the K axis (positions >= klen read as zero)
    __device__ __forceinline__ void init (const ActView<COH> &v, uint32_t first, uint32_t ld_, uint32_t valid_rows, uint32_t klen_, uint32_t tid)
    {
        view = v; ld = ld_; klen = klen_; c4 = tid & 15; s0 = tid >> 4; live = c4 * 4 < valid_rows;
        off[0] = first + s0 * ld + c4 * 4;
        off[1] = first + (s0 + 16) * ld + c4 * 4;
    }
    __device__ __forceinline__ void load (int it, float4 (&v)[2])
    {
        const float4 z = make_float4 (0.f, 0.f, 0.f, 0.f);
        const uint32_t s = it * GEMM_BK + s0;
        v[0] = (live && s < klen) ? view.ld4 (off[0] + it * GEMM_BK * ld) : z;
        v[1] = (live && s + 16 < klen) ? view.ld4 (off[1] + it * GEMM_BK * ld) : z;
    }
    __device__ __forceinline__ void store (float *lds, const float4 (&v)[2])
    {
        #pragma unroll
        for (int i = 0; i < 2; i++)
        {
            float *d = lds + (c4 * 4) * LDS_ROW + s0 + 16 * i;
            d[0] = v[i].x; d[LDS_ROW] = v[i].y; d[2 * LDS_ROW] = v[i].z; d[3 * LDS_ROW] = v[i].w;
        }
    }
};

// ---------------------------------------------------------------------------------------------
// fp32 MFMA core.  Workgroup tile = BM weight rows x BN activation rows; WM x WN wavefronts, each
// owning (BM/WM) x (BN/WN) built from 32x32 v_mfma_f32_32x32x2_f32 blocks.  The activation row is
// the MFMA row index and the weight row the MFMA column, so each accumulator register holds 32
// consecutive output channels of one output column: stores are 128-byte coalesced.
// One LDS stage; the K slice after the staged one waits in registers.
// ---------------------------------------------------------------------------------------------
// LDS-only barrier: waits for this wave's LDS traffic, not for global loads still in flight.
// The thread index as a value the optimiser cannot move out of an enclosing persistent loop: the
// per-lane address arithmetic of every tile kind is loop-invariant there, would be hoisted in front of
// the loop and then be kept alive (spilled to scratch) across all tiles.
__device__ __forceinline__ uint32_t tile_thread ()
{
    uint32_t t = threadIdx.x;
    asm volatile ("" : "+v"(t));
    return t & (WG_THREADS - 1);
}

__device__ __forceinline__ void lds_barrier ()
{
    asm volatile ("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Instruction-group hints for the machine scheduler (masks of __builtin_amdgcn_sched_group_barrier)
#define SG_MFMA 0x008
#define SG_VMEM_READ 0x020
#define SG_DS_READ 0x100
#define SG_DS_WRITE 0x200

// DEPTH = number of K slices in flight from memory (register sets): 1 = the slice after the staged one
// waits in registers; 2 = the two slices after it do.  A slice cannot take less than the memory latency
// divided by DEPTH, and when a compute unit runs fewer workgroups than it could hold (a graph bound by its
// dependency chains) nothing else hides that latency; the second set costs 4 registers per 32 operand rows.
// Instruction-arbiter priority of a wavefront everywhere but inside a K loop.  The workgroups of a compute unit share
// its matrix pipeline; the ones in a K loop can keep it busy by themselves, while a workgroup in a tile's set-up,
// first operand fetch, epilogue or scheduling step is on the graph's critical path with a handful of instructions:
// those go first, and the K loops fill every slot they leave.  (The opposite order, K loops first, is slower than
// no priorities at all.)
#define TILE_PRIO 2
struct NoHook { __device__ __forceinline__ void operator() () const {} };

// What a kernel that runs tiles is compiled for.  The persistent kernel exists in a few variants that leave out the
// tile kinds a graph does not contain: four workgroups in different phases share a compute unit's 64 KB instruction
// cache, and a transformer graph has no use for the convolution loaders' K loops, nor a ResNet for the attention tiles.
enum : unsigned
{
    TILES_GATHER = 1u,          // contraction operands gathered through ConvLoader (convolutions, FC layers over images)
    TILES_LARGE = 2u, TILES_WIDE = 4u, TILES_SMALL = 8u,       // contraction tile shapes
    TILES_ATTENTION = 16u, TILES_NORM = 32u /* layernorm, softmax */, TILES_POOL = 64u, TILES_YOLO = 128u /* yolo, append */,
    TILES_RESIDUAL = 256u,
    TILES_NARROW = 512u,        // the 32 x 32 contraction tile of latency-bound graphs
    TILES_TALL = 1024u,         // the 128 x 32 contraction tile of weight-streaming layers
    TILES_ALL = 2047u,
    TILES_CONVNET = TILES_GATHER | TILES_LARGE | TILES_WIDE | TILES_SMALL | TILES_POOL | TILES_RESIDUAL,
    TILES_TRANSFORMER = TILES_SMALL | TILES_ATTENTION | TILES_NORM | TILES_RESIDUAL
};
// `before_last_slice` runs right before the MFMAs of the last K slice: the place to request what the epilogue
// will need from memory, with the operand registers free and a whole slice of arithmetic to hide the latency.
// `ready` runs between the first request for the weight operand and the first request for the activation operand: a
// kernel that starts tiles before their parents have finished (see the ordered mode of the persistent kernel) waits
// there, with the tile's set-up done and its first weights on their way.
template <int BM, int BN, int WM, int WN, int DEPTH, class ALoader, class BLoader, class Hook = NoHook, class Ready = NoHook>
__device__ __forceinline__ void gemm_core (ALoader &al, BLoader &bl, int kbase, int kiters, float *smem,
    floatx16 (&acc)[BN / WN / 32][BM / WM / 32], bool phases = false, Hook before_last_slice = Hook (), Ready ready = Ready ())
{
    static_assert (DEPTH == 1 || DEPTH == 2, "one or two register sets");
    if (phases) tile_phase_lap (12);
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr int KK = GEMM_BK / 8;
    const uint32_t tid = tile_thread (), lane = tid & 63, wave = tid >> 6;
    const uint32_t wm0 = (wave % WM) * (BM / WM), wn0 = (wave / WM) * (BN / WN);
    const float *afrag = smem + wm0 * LDS_ROW + (lane & 31) * LDS_ROW + (lane >> 5) * 4;
    const float *bfrag = smem + BM * LDS_ROW + wn0 * LDS_ROW + (lane & 31) * LDS_ROW + (lane >> 5) * 4;

    #pragma unroll
    for (int i = 0; i < TN; i++)
        #pragma unroll
        for (int j = 0; j < TM; j++)
            #pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    // fragments of sub-step s (8 K values: lanes 0-31 take the first four, lanes 32-63 the last four)
    float4 af[2][TM], bf[2][TN];
    auto read_frags = [&] (int buf, int sub)
    {
        #pragma unroll
        for (int j = 0; j < TM; j++) af[buf][j] = ld4 (afrag + j * 32 * LDS_ROW + sub * 8);
        #pragma unroll
        for (int i = 0; i < TN; i++) bf[buf][i] = ld4 (bfrag + i * 32 * LDS_ROW + sub * 8);
    };
    // half = 0: K components x, y of the fragments; half = 1: z, w
    auto mfma_half = [&] (int buf, int half)
    {
        #pragma unroll
        for (int i = 0; i < TN; i++)
            #pragma unroll
            for (int j = 0; j < TM; j++)
            {
                if (half == 0)
                {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32 (bf[buf][i].x, af[buf][j].x, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32 (bf[buf][i].y, af[buf][j].y, acc[i][j], 0, 0, 0);
                }
                else
                {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32 (bf[buf][i].z, af[buf][j].z, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32 (bf[buf][i].w, af[buf][j].w, acc[i][j], 0, 0, 0);
                }
            }
    };

    // register set s holds slice it with (it - first) % DEPTH == s
    float4 areg[DEPTH][ALoader::R], breg[DEPTH][BLoader::R];
    al.load (kbase, areg[0]); ready (); bl.load (kbase, breg[0]);
    if (DEPTH == 2 && kiters > 1) { al.load (kbase + 1, areg[DEPTH - 1]); bl.load (kbase + 1, breg[DEPTH - 1]); }
    al.store (smem, areg[0]); bl.store (smem + BM * LDS_ROW, breg[0]);
    if (kiters > DEPTH) { al.load (kbase + DEPTH, areg[0]); bl.load (kbase + DEPTH, breg[0]); }
    lds_barrier ();
    if (phases) tile_phase_lap (8);
    __builtin_amdgcn_s_setprio (0);
    read_frags (0, 0);

    // One K slice per iteration, single LDS stage, software-pipelined by hand:
    //   sub-steps 0 .. KK-2: the fragments of sub-step s+1 are fetched between the two halves of the
    //   MFMAs of sub-step s, so they have arrived even if the compiler waits for ALL LDS traffic before s+1;
    //   last sub-step: once every wave holds its last fragments (barrier), the next slice (waiting in
    //   registers) overwrites the stage and the slice DEPTH after it is requested from memory into the
    //   registers just freed, all under the first half of the sub-step's MFMAs; after the second barrier the
    //   first fragments of the new slice are fetched under the second half.
    // The scheduling-group hints pin that order; left alone, the compiler fetches each fragment right
    // before its use and the LDS latency shows.
    // `set` (a literal at every call, so that the register arrays are indexed statically) = the register set
    // that holds slice it + 1.
    auto slice = [&] (int it, int set)
    {
        #pragma unroll
        for (int kk = 0; kk + 1 < KK; kk++)
        {
            mfma_half (kk & 1, 0);
            read_frags ((kk + 1) & 1, kk + 1);
            mfma_half (kk & 1, 1);
            __builtin_amdgcn_sched_group_barrier (SG_MFMA, 2 * TM * TN, 0);
            __builtin_amdgcn_sched_group_barrier (SG_DS_READ, TM + TN, 0);
            __builtin_amdgcn_sched_group_barrier (SG_MFMA, 2 * TM * TN, 0);
        }
        __builtin_amdgcn_sched_barrier (0);
        lds_barrier ();
        __builtin_amdgcn_sched_barrier (0);
        al.store (smem, areg[set]); bl.store (smem + BM * LDS_ROW, breg[set]);
        if (DEPTH == 2)
        {
            // always issued (the last slices are requested again and never used): a request inside a branch makes
            // the compiler lose count of what is in flight, and it then waits for everything before every store
            const int nxt = kbase + min (it + 1 + DEPTH, kiters - 1);
            al.load (nxt, areg[set]); bl.load (nxt, breg[set]);
        }
        else if (it + 1 + DEPTH < kiters) { al.load (kbase + it + 1 + DEPTH, areg[set]); bl.load (kbase + it + 1 + DEPTH, breg[set]); }
        mfma_half ((KK - 1) & 1, 0);
        __builtin_amdgcn_sched_barrier (0);
        lds_barrier ();
        __builtin_amdgcn_sched_barrier (0);
        read_frags (0, 0);
        mfma_half ((KK - 1) & 1, 1);
        __builtin_amdgcn_sched_group_barrier (SG_DS_READ, TM + TN, 0);
        __builtin_amdgcn_sched_group_barrier (SG_MFMA, 2 * TM * TN, 0);
    };
    if (DEPTH == 1)
        for (int it = 0; it + 1 < kiters; it++) slice (it, 0);
    else
    {
        // slice it + 1 sits in set (it + 1) % 2: two slices per trip keep the set a literal
        int it = 0;
        for (; it + 2 < kiters; it += 2) { slice (it, DEPTH - 1); slice (it + 1, 0); }
        if (it + 1 < kiters) slice (it, DEPTH - 1);
    }
    // last slice: nothing left to stage
    before_last_slice ();
    #pragma unroll
    for (int kk = 0; kk < KK; kk++)
    {
        mfma_half (kk & 1, 0);
        if (kk + 1 < KK) read_frags ((kk + 1) & 1, kk + 1);
        mfma_half (kk & 1, 1);
        __builtin_amdgcn_sched_group_barrier (SG_MFMA, 2 * TM * TN, 0);
        if (kk + 1 < KK) __builtin_amdgcn_sched_group_barrier (SG_DS_READ, TM + TN, 0);
        __builtin_amdgcn_sched_group_barrier (SG_MFMA, 2 * TM * TN, 0);
    }
    __builtin_amdgcn_s_setprio (TILE_PRIO);
    lds_barrier ();          // the caller reuses the stage (epilogue)
}

// The same for the 64 x 64 shape, whose four waves own ONE 32 x 32 block each, scheduled by hand for a
// workgroup that has its compute unit (nearly) to itself -- the normal case for these tiles: they are the
// short tiles of layers cut along K, and in a graph bound by its dependency chains only one or two
// workgroups per compute unit are inside a K loop at any time.  Then nothing but this wave's own instruction
// order hides the slice boundary (two barriers, the LDS refill, the next requests): in gemm_core the matrix
// pipeline drains there, 16 MFMAs of 64 cycles each took ~1600 cycles per slice.
// Here the fragments of all four sub-steps of a slice are resident (8 registers each, affordable with one
// accumulator block), so every piece of boundary work sits between two MFMAs that do not depend on it:
//   M00 M01 M02 |X| M03 wA M10 wB M11 gA M12 gB M13 M20 |Y| M21 r0 M22 r1 M23 M30 r2 M31 M32 M33 r3
// Mij = MFMA on K pair j of sub-step i; X = barrier "everyone holds this slice's fragments", wA / wB = next
// slice registers -> LDS, gA / gB = requests for the slice DEPTH ahead, Y = barrier "refill visible",
// ri = fragments of sub-step i of the next slice (its buffer was released by Mi3).
// Accumulator register v of MFMA block (i, j) holds output (row n, channel m):
//   n = wn0 + 32 i + 8 (v / 4) + 4 (lane / 32) + v % 4,   m = wm0 + 32 j + lane % 32
#define ACC_N(wn0, i, v, lane) ((wn0) + 32 * (i) + 8 * ((v) >> 2) + 4 * ((lane) >> 5) + ((v) & 3))

struct NoStats { __device__ __forceinline__ void operator() (const float4 (&)[2]) const {} };

// A layer norm folded into a matmul tile (aspen_hip_layer_t.norm_fold), second half: the K loop has left every thread
// the sum and the sum of squares of its eight-th of two columns' K axis (thread t: columns t / 8 and t / 8 + 32, the
// ActRowLoader's assignment).  The eight threads of a column add up, one of them writes the column's mean and
// 1 / sqrt (variance + eps) behind the stage in LDS, and every lane corrects its sixteen sums:
// acc = rstd[n] * (acc - mean[n] * rowsum[m]).  Same arithmetic for mean and variance as tile_layernorm.
#define NORM_FOLD_STATS_OFFSET (128 * LDS_ROW)      // floats: behind the two operand blocks of the stage
template <int COH>
__device__ __forceinline__ void norm_fold_finish (const aspen_hip_layer_t &L, floatx16 &acc, float (&cs)[2], float (&cq)[2], float *smem,
    uint32_t tid, uint32_t m0, uint32_t n0, uint32_t wm0, uint32_t wn0)
{
    const uint32_t lane = tid & 63;
    #pragma unroll
    for (int o = 1; o < 8; o <<= 1)
    {
        #pragma unroll
        for (int i = 0; i < 2; i++) { cs[i] += __shfl_xor (cs[i], o, 64); cq[i] += __shfl_xor (cq[i], o, 64); }
    }
    float *st = smem + NORM_FOLD_STATS_OFFSET;
    if ((tid & 7u) == 0)
    {
        #pragma unroll
        for (int i = 0; i < 2; i++)
        {
            const float mean = cs[i] / (float)L.K;
            const float var = cq[i] / (float)L.K - mean * mean;
            const uint32_t n = (tid >> 3) + 32 * i;
            const float rstd = 1.0f / sqrtf (var + 1e-6f);
            st[2 * n] = mean; st[2 * n + 1] = rstd;
            // (row 0 of the layer that was asked to: the pairs go to memory as well, for a fused shortcut that needs the
            // normalised matrix nobody writes any more)
            if (L.norm_stats != nullptr && m0 == 0 && n0 + n < L.N)
            {
                ActView<COH> sv;
                sv.init (L.norm_stats, L.N, 2);
                sv.st1 (2 * (n0 + n), mean); sv.st1 (2 * (n0 + n) + 1, rstd);
            }
        }
    }
    // (the row sums are weights: requested before the barrier)
    const uint32_t m = min (m0 + wm0 + (lane & 31), L.M - 1);
    const float rs = gld1 (L.in1 + m);
    lds_barrier ();
    #pragma unroll
    for (int v = 0; v < 16; v++)
    {
        const uint32_t n = ACC_N (wn0, 0, v, lane);
        acc[v] = st[2 * n + 1] * (acc[v] - st[2 * n] * rs);
    }
}

template <int DEPTH, class ALoader, class BLoader, class Hook = NoHook, class Ready = NoHook, class Stats = NoStats>
__device__ __forceinline__ void gemm_core_single_block (ALoader &al, BLoader &bl, int kbase, int kiters, float *smem,
    floatx16 (&accs)[1][1], bool phases = false, Hook before_last_slice = Hook (), Ready ready = Ready (), Stats stats = Stats ())
{
    // `stats` sees every K slice of the activation operand once, as the registers it passes through on its way into LDS
    // (a folded layer norm's column sums, see norm_fold_finish)
    static_assert (DEPTH == 1 || DEPTH == 2, "one or two register sets");
    static_assert (ALoader::R == 2 && BLoader::R == 2 && GEMM_BK == 32, "64 x 64 tile, four sub-steps");
    constexpr int BM = 64;
    if (phases) tile_phase_lap (12);
    const uint32_t tid = tile_thread (), lane = tid & 63, wave = tid >> 6;
    const uint32_t wm0 = (wave % 2) * 32, wn0 = (wave / 2) * 32;
    const float *afrag = smem + wm0 * LDS_ROW + (lane & 31) * LDS_ROW + (lane >> 5) * 4;
    const float *bfrag = smem + BM * LDS_ROW + wn0 * LDS_ROW + (lane & 31) * LDS_ROW + (lane >> 5) * 4;
    floatx16 acc;
    #pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = 0.f;
    float4 fa[4], fb[4];
#define SB __builtin_amdgcn_sched_barrier (0)
#define RD(i) do { fa[i] = ld4 (afrag + (i) * 8); fb[i] = ld4 (bfrag + (i) * 8); SB; } while (0)
#define MF(i, c) do { acc = __builtin_amdgcn_mfma_f32_32x32x2f32 (fb[i].c, fa[i].c, acc, 0, 0, 0); SB; } while (0)
    float4 areg[DEPTH][2], breg[DEPTH][2];
    al.load (kbase, areg[0]); ready (); bl.load (kbase, breg[0]);
    if (DEPTH == 2 && kiters > 1) { al.load (kbase + 1, areg[DEPTH - 1]); bl.load (kbase + 1, breg[DEPTH - 1]); }
    al.store (smem, areg[0]); bl.store (smem + BM * LDS_ROW, breg[0]); stats (breg[0]);
    if (kiters > DEPTH) { al.load (kbase + DEPTH, areg[0]); bl.load (kbase + DEPTH, breg[0]); }
    lds_barrier ();
    if (phases) tile_phase_lap (8);
    __builtin_amdgcn_s_setprio (0);
    SB; RD (0); RD (1); RD (2); RD (3);
    // `set` (a literal at every call) = the register set that holds slice it + 1
    auto slice = [&] (int it, int set)
    {
        // requests are always issued (the last slices are asked for again and never used): a request inside a
        // branch makes the compiler lose count of what is in flight, and it then waits for everything
        const int nxt = kbase + (DEPTH == 2 ? min (it + 1 + DEPTH, kiters - 1) : it + 2);
        SB; MF (0, x); MF (0, y); MF (0, z);
        lds_barrier (); SB;
        MF (0, w); al.store (smem, areg[set]); SB;
        MF (1, x); bl.store (smem + BM * LDS_ROW, breg[set]); stats (breg[set]); SB;
        MF (1, y); if (DEPTH == 2 || it + 2 < kiters) al.load (nxt, areg[set]); SB;
        MF (1, z); if (DEPTH == 2 || it + 2 < kiters) bl.load (nxt, breg[set]); SB;
        MF (1, w); MF (2, x);
        lds_barrier (); SB;
        MF (2, y); RD (0);
        MF (2, z); RD (1);
        MF (2, w); MF (3, x); RD (2);
        MF (3, y); MF (3, z); MF (3, w); RD (3);
    };
    if (DEPTH == 1)
        for (int it = 0; it + 1 < kiters; it++) slice (it, 0);
    else
    {
        int it = 0;
        for (; it + 2 < kiters; it += 2) { slice (it, DEPTH - 1); slice (it + 1, 0); }
        if (it + 1 < kiters) slice (it, DEPTH - 1);
    }
    before_last_slice ();
    SB;
    MF (0, x); MF (0, y); MF (0, z); MF (0, w); MF (1, x); MF (1, y); MF (1, z); MF (1, w);
    MF (2, x); MF (2, y); MF (2, z); MF (2, w); MF (3, x); MF (3, y); MF (3, z); MF (3, w);
#undef SB
#undef RD
#undef MF
    accs[0][0] = acc;
    __builtin_amdgcn_s_setprio (TILE_PRIO);
    lds_barrier ();          // the caller reuses the stage (epilogue)
}


// Shortcut fused into a contraction epilogue: fuse_out = fuse_act (v + fuse_in) for the (up to) four
// channels m .. m+3 of column n; `left` = channels of the matrix from m on.  Same arithmetic, in the same
// order, as a residual tile reading the stored v would do.
template <int COH>
__device__ __forceinline__ void fused_shortcut (const aspen_hip_layer_t &L, const ActView<COH> &fin, const ActView<COH> &fout,
    float4 v, uint32_t n, uint32_t m, uint32_t left)
{
    const uint32_t oi = n * L.fuse_ld_in + m, oo = n * L.ld + m;
    if (left >= 4)
    {
        const float4 s = fin.ld4 (oi);
        v.x += s.x; v.y += s.y; v.z += s.z; v.w += s.w;
        fout.st4 (oo, act4 (v, L.fuse_act));
    }
    else
    {
        fout.st1 (oo, activate (v.x + fin.ld1 (oi), L.fuse_act));
        if (left > 1) fout.st1 (oo + 1, activate (v.y + fin.ld1 (oi + 1), L.fuse_act));
        if (left > 2) fout.st1 (oo + 2, activate (v.z + fin.ld1 (oi + 2), L.fuse_act));
    }
}

// conv / FC / matmul tile
// `slice` < 0: the whole K axis, bias + activation, result to the layer's matrix.  `slice` >= 0 (split-K):
// K slices [slice*kiters_per_split, ...) only, raw sums to that slice's partial matrix.
// This part (operand loaders, K loop, accumulators parked in LDS) exists once per tile shape; the
// epilogue that follows it is shared by all shapes, which keeps the kernel's code small.
// what the main loop already requested for the epilogue (threads whose four channels all exist): the bias, and all
// of the thread's pieces of a fused shortcut's operand (a tile has at most 128 columns: 8 pieces per thread)
struct shortcut_prefetch_t { float4 s[8]; float4 bias; bool have, have_shortcut; };

template <int BM, int BN, int WM, int WN, int DEPTH, int COH, unsigned FEAT, class Descriptor, class Ready>
__device__ __forceinline__ void contraction_mainloop (const aspen_hip_layer_t &L, Descriptor descriptor, uint32_t tn, uint32_t tm, int slice, float *smem, shortcut_prefetch_t &pre, Ready ready)
{
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr bool SINGLE = TM * TN == 1 && BM == VAR2_BM && BN == VAR2_BN;     // the hand-scheduled loop of the 64 x 64 shape
    const uint32_t tid = tile_thread (), lane = tid & 63, wave = tid >> 6;
    const uint32_t m0 = tm * BM, n0 = tn * BN;
    floatx16 acc[TN][TM];
    ActView<COH> in;
    // (the operands' addresses come from loads of their own: taken from `L` they are parts of an 8-register piece of
    // the descriptor, which the compiler then keeps alive, spills and restores as a whole around every K slice)
    in.init (descriptor ().in0, L.in0_columns, L.ld0);
    int kbase = 0, kiters = (int)(L.Kp / GEMM_BK);
    if (slice >= 0)
    {
        kbase = slice * (int)L.kiters_per_split;
        kiters = min ((int)L.kiters_per_split, kiters - kbase);
    }
    RowLoader<BM> al;
    al.init (descriptor ().weight, m0, (L.M + 127u) / 128u * 128u, L.Kp, tid);
    // a fused shortcut's other operand comes from memory another XCD may have written: the first pieces this
    // thread will need in the epilogue (see contraction_epilogue for the thread -> piece mapping) are
    // requested under the last K slice
    // (`L` below is a fresh copy of the descriptor: what only this hook needs stays out of the K loop's registers)
    auto fetch_shortcut = [&] ()
    {
        const aspen_hip_layer_t L = descriptor ();
        constexpr uint32_t C4_LOG2 = BM == 128 ? 5 : 4, STEP = WG_THREADS >> C4_LOG2, PIECES = BN / STEP;
        static_assert (PIECES <= 8, "pieces per thread");
        const uint32_t c = (tid & ((1u << C4_LOG2) - 1)) * 4, rows = min ((uint32_t)BN, L.N - n0), r0 = tid >> C4_LOG2;
        pre.have = slice < 0 && c + 4 <= L.M - m0;
        pre.have_shortcut = pre.have && L.fuse_out != nullptr;
        if (pre.have) pre.bias = L.bias ? gld4 (L.bias + m0 + c) : make_float4 (0.f, 0.f, 0.f, 0.f);
        if (pre.have_shortcut)
        {
            ActView<COH> fin;
            fin.init (L.fuse_in, L.N, L.fuse_ld_in);
            #pragma unroll
            for (uint32_t u = 0; u < PIECES; u++)
                if (r0 + u * STEP < rows) pre.s[u] = fin.ld4 ((n0 + r0 + u * STEP) * L.fuse_ld_in + m0 + c);
        }
    };
    if (L.direct == ASPEN_HIP_OPERAND_DIRECT)
    {
        ActRowLoader<BN, COH> bl;
        bl.init (in, n0, L.N - 1, L.ld0, 0, tid);
        if constexpr (SINGLE && (FEAT & TILES_NORM) != 0)
        {
            // (kernels for transformer graphs: the column sums a folded layer norm needs are gathered in every such tile,
            // sixteen additions and multiplications per K slice, and used where the layer asks for them)
            float cs[2] = {0.f, 0.f}, cq[2] = {0.f, 0.f};
            auto stats = [&] (const float4 (&b)[2])
            {
                #pragma unroll
                for (int i = 0; i < 2; i++)
                {
                    cs[i] += (b[i].x + b[i].y) + (b[i].z + b[i].w);
                    cq[i] += (b[i].x * b[i].x + b[i].y * b[i].y) + (b[i].z * b[i].z + b[i].w * b[i].w);
                }
            };
            gemm_core_single_block<DEPTH> (al, bl, kbase, kiters, smem, acc, COH != 0, fetch_shortcut, ready, stats);
            if (L.norm_fold) norm_fold_finish<COH> (L, acc[0][0], cs, cq, smem, tid, m0, n0, (wave % 2) * 32, (wave / 2) * 32);
        }
        else if constexpr (SINGLE) gemm_core_single_block<DEPTH> (al, bl, kbase, kiters, smem, acc, COH != 0, fetch_shortcut, ready);
        else gemm_core<BM, BN, WM, WN, DEPTH> (al, bl, kbase, kiters, smem, acc, COH != 0, fetch_shortcut, ready);
    }
    else if constexpr ((FEAT & TILES_GATHER) != 0)
    {
        // (the dense three-channel layout is only used for layers of up to 64 output channels, see aspen_layer_dense3)
        if (BM == 64 && L.direct == ASPEN_HIP_OPERAND_DENSE3)
        {
            Dense3Loader<BN, COH> bl;
            bl.init (L, in, n0, tid);
            if constexpr (SINGLE) gemm_core_single_block<DEPTH> (al, bl, kbase, kiters, smem, acc, COH != 0, fetch_shortcut, ready);
            else gemm_core<BM, BN, WM, WN, DEPTH> (al, bl, kbase, kiters, smem, acc, COH != 0, fetch_shortcut, ready);
        }
        else if (SINGLE && L.IC % GEMM_BK != 0)
        {
            if constexpr (SINGLE)
            {
                ConvLoader<BN, COH, true> bl;
                bl.init (L, in, n0, tid, kbase);
                gemm_core_single_block<DEPTH> (al, bl, kbase, kiters, smem, acc, COH != 0, fetch_shortcut, ready);
            }
        }
        else
        {
            ConvLoader<BN, COH, false> bl;
            bl.init (L, in, n0, tid, kbase);
            if constexpr (SINGLE) gemm_core_single_block<DEPTH> (al, bl, kbase, kiters, smem, acc, COH != 0, fetch_shortcut, ready);
            else gemm_core<BM, BN, WM, WN, DEPTH> (al, bl, kbase, kiters, smem, acc, COH != 0, fetch_shortcut, ready);
        }
    }
    if (COH) tile_phase_lap (9);
    const uint32_t wm0 = (wave % WM) * (BM / WM), wn0 = (wave / WM) * (BN / WN);
    if (slice >= 0)
    {
        // split-K: the raw sums go straight from the accumulators to this slice's block of the output tile, in the
        // accumulators' own layout (splitk_gather reads them back the same way): four 16-byte stores per lane, each
        // instruction 1 KB in one piece; no bias, no activation, no bounds, nothing to stage through LDS.  Only the
        // 64 x 64 and the 128 x 32 shape (one accumulator block per wavefront either way) are ever cut along K.
        if constexpr (TM * TN == 1)
        {
            const aspen_hip_layer_t L = descriptor ();
            const uint32_t tiles = L.tiles_m * L.tiles_n;
            ActView<COH> part;
            part.init (L.partial, L.splits * tiles, SPLITK_TILE_FLOATS);
            const uint32_t base = ((uint32_t)slice * tiles + tn * L.tiles_m + tm) * SPLITK_TILE_FLOATS + tid * 4;
            #pragma unroll
            for (int q = 0; q < 4; q++)
                part.st4 (base + q * 4 * WG_THREADS, make_float4 (acc[0][0][4 * q], acc[0][0][4 * q + 1], acc[0][0][4 * q + 2], acc[0][0][4 * q + 3]));
        }
        return;
    }
    // Epilogue through LDS (free after the last K slice): the raw accumulators are parked as
    // [column][channel] for contraction_epilogue.
    constexpr int TROW = BM + 8;            // (4 * TROW) % 64 == 32: the two half-waves hit disjoint banks
    #pragma unroll
    for (int j = 0; j < TM; j++)
        #pragma unroll
        for (int i = 0; i < TN; i++)
            #pragma unroll
            for (int v = 0; v < 16; v++)
                smem[ACC_N (wn0, i, v, lane) * TROW + wm0 + 32 * j + (lane & 31)] = acc[i][j][v];
    __syncthreads ();
}

// Second part of a contraction tile of BM = 4 << c4_log2 channels by BN columns, accumulators parked in
// LDS as [column][BM + 8]: a rolled loop adds the bias, applies the activation and writes 128-bit pieces,
// so a wavefront covers whole 512-byte (BM = 128) / 256-byte (BM = 64) runs of a column.
template <int COH, bool NORM = false>
__device__ __forceinline__ void contraction_epilogue (const aspen_hip_layer_t &L, uint32_t tn, uint32_t tm, float *smem,
    uint32_t c4_log2, uint32_t BN, const shortcut_prefetch_t &pre)
{
    const uint32_t tid = tile_thread ();
    const uint32_t C4 = 1u << c4_log2, BM = 4u << c4_log2, TROW = BM + 8;
    const uint32_t m0 = tm * BM, n0 = tn * BN;
    const int act = L.act;
    ActView<COH> out;
    out.init (L.out, L.N, L.ld);
    const uint32_t rows = min (BN, L.N - n0);
    const uint32_t mrem = L.M - m0;         // channels of this tile that exist (may exceed BM)
    const uint32_t c = (tid & (C4 - 1)) * 4;      // WG_THREADS is a multiple of C4: a thread keeps its channels
    if (c < mrem)
    {
        float4 b = make_float4 (0.f, 0.f, 0.f, 0.f);
        if (pre.have) b = pre.bias;
        else if (L.bias)
        {
            if (c + 4 <= mrem) b = gld4 (L.bias + m0 + c);
            else { b.x = gld1 (L.bias + m0 + c); if (c + 1 < mrem) b.y = gld1 (L.bias + m0 + c + 1); if (c + 2 < mrem) b.z = gld1 (L.bias + m0 + c + 2); }
        }
        const bool fuse = L.fuse_out != nullptr;
        const bool keep = !(fuse && L.fuse_discard);        // the pre-shortcut sums are stored unless the host has no use for them
        ActView<COH> fin, fout;
        if (fuse) { fin.init (L.fuse_in, L.N, L.fuse_ld_in); fout.init (L.fuse_out, L.N, L.ld); }
        // the shortcut's operand may be the input of a layer norm nobody runs as a layer any more: normalised here, with
        // the arithmetic of tile_layernorm (see aspen_hip_layer_t.fuse_norm_stats)
        const bool normed = NORM && fuse && L.fuse_norm_stats != nullptr;
        ActView<COH> stv;
        float4 gam = make_float4 (1.f, 1.f, 1.f, 1.f), bet = make_float4 (0.f, 0.f, 0.f, 0.f);
        if (NORM && normed)
        {
            stv.init (L.fuse_norm_stats, L.N, 2);
            gam = gld4 (L.fuse_norm_gamma + m0 + c);
            if (L.fuse_norm_beta) bet = gld4 (L.fuse_norm_beta + m0 + c);
        }
        const uint32_t STEP = WG_THREADS >> c4_log2;
        constexpr uint32_t U = 4;                              // 4 rows at a time: all 8 of the larger tiles measured slower (code size, registers)
        if (c + 4 <= mrem)
        {
            // whole float4 of channels: rows are handled U at a time, all LDS reads and shortcut loads of a
            // group issued before its first store.  Loads and stores share one in-order counter, so a
            // shortcut load issued after a (write-through) store waits for that store's acknowledgement.
            // The shortcut pieces were requested under the last K slice (pre); group g's are pre.s[4 g ..].
            #pragma unroll
            for (uint32_t g = 0; g < 2; g++)
            {
                const uint32_t r0 = (tid >> c4_log2) + g * U * STEP;
                if (r0 >= rows) break;
                float4 v[U], s[U];
                float mu[U], rs[U];
                #pragma unroll
                for (uint32_t u = 0; u < U; u++)
                {
                    const uint32_t r = r0 + u * STEP;
                    if (r < rows)
                    {
                        v[u] = ld4 (smem + r * TROW + c);
                        if (fuse) s[u] = pre.have_shortcut ? pre.s[g * U + u] : fin.ld4 ((n0 + r) * L.fuse_ld_in + m0 + c);
                        if (NORM && normed) { mu[u] = stv.ld1 (2 * (n0 + r)); rs[u] = stv.ld1 (2 * (n0 + r) + 1); }
                    }
                }
                #pragma unroll
                for (uint32_t u = 0; u < U; u++)
                {
                    const uint32_t r = r0 + u * STEP;
                    if (r < rows)
                    {
                        float4 y = v[u];
                        y.x += b.x; y.y += b.y; y.z += b.z; y.w += b.w;
                        y = act4 (y, act);
                        const uint32_t o = (n0 + r) * L.ld + m0 + c;
                        if (keep) out.st4 (o, y);
                        if (fuse)
                        {
                            if (NORM && normed)
                            {
                                s[u].x = (s[u].x - mu[u]) * rs[u] * gam.x + bet.x; s[u].y = (s[u].y - mu[u]) * rs[u] * gam.y + bet.y;
                                s[u].z = (s[u].z - mu[u]) * rs[u] * gam.z + bet.z; s[u].w = (s[u].w - mu[u]) * rs[u] * gam.w + bet.w;
                            }
                            y.x += s[u].x; y.y += s[u].y; y.z += s[u].z; y.w += s[u].w;
                            fout.st4 (o, act4 (y, L.fuse_act));
                        }
                    }
                }
            }
        }
        else
            for (uint32_t r = tid >> c4_log2; r < rows; r += STEP)      // last, partial group of channels
            {
                float4 v = ld4 (smem + r * TROW + c);
                v.x += b.x; v.y += b.y; v.z += b.z; v.w += b.w;
                v = act4 (v, act);
                const uint32_t o = (n0 + r) * L.ld + m0 + c;
                if (keep) { out.st1 (o, v.x); if (c + 1 < mrem) out.st1 (o + 1, v.y); if (c + 2 < mrem) out.st1 (o + 2, v.z); }
                if (fuse) fused_shortcut<COH> (L, fin, fout, v, n0 + r, m0 + c, mrem - c);
            }
    }
    // no barrier here: whatever runs next on this workgroup (the scheduling step of the persistent kernel) passes
    // one before LDS is written again
}

// split-K, run by the slice that finishes last: the sum of the slices' blocks (in slice order, whoever runs it) in
// the accumulator layout they were stored in, parked in LDS as [column][channel] like the accumulators of an unsplit
// tile, so that contraction_epilogue finishes both alike.  Eight 16-byte loads in flight per thread: their memory
// latencies overlap instead of adding up (the blocks come from other XCDs' tiles and miss this XCD's L2); a slice
// index past the last one re-reads the last slice and is not added.
template <int COH>
__device__ __forceinline__ void splitk_gather (const aspen_hip_layer_t &L, uint32_t t, float *smem, bool tall = false)
{
    const uint32_t tid = tile_thread (), lane = tid & 63, wave = tid >> 6;
    const uint32_t tiles = L.tiles_m * L.tiles_n, sstride = tiles * SPLITK_TILE_FLOATS, last = L.splits - 1;
    ActView<COH> part;
    part.init (L.partial, L.splits * tiles, SPLITK_TILE_FLOATS);
    const uint32_t base = t * SPLITK_TILE_FLOATS + tid * 4;
    constexpr uint32_t BATCH = 2;       // (1 and 4 measured: no better)
    float4 v[4];
    #pragma unroll
    for (int q = 0; q < 4; q++) v[q] = make_float4 (0.f, 0.f, 0.f, 0.f);
    for (uint32_t s0 = 0; s0 < L.splits; s0 += BATCH)
    {
        float4 p[BATCH][4];
        #pragma unroll
        for (uint32_t j = 0; j < BATCH; j++)
            #pragma unroll
            for (int q = 0; q < 4; q++) p[j][q] = part.ld4 (base + min (s0 + j, last) * sstride + q * 4 * WG_THREADS);
        #pragma unroll
        for (uint32_t j = 0; j < BATCH; j++)
        {
            const bool use = s0 + j <= last;
            #pragma unroll
            for (int q = 0; q < 4; q++)
            { v[q].x += use ? p[j][q].x : 0.f; v[q].y += use ? p[j][q].y : 0.f; v[q].z += use ? p[j][q].z : 0.f; v[q].w += use ? p[j][q].w : 0.f; }
        }
    }
    // (tall: 128 channels x 32 columns, the four wavefronts' blocks below each other; else 2 x 2 blocks of 64 x 64)
    const uint32_t TROW = (tall ? VAR4_BM : VAR2_BM) + 8;
    const uint32_t wm0 = tall ? wave * 32 : (wave % 2) * 32, wn0 = tall ? 0u : (wave / 2) * 32, m = wm0 + (lane & 31);
    #pragma unroll
    for (int q = 0; q < 4; q++)
    {
        smem[ACC_N (wn0, 0, 4 * q, lane) * TROW + m] = v[q].x;
        smem[ACC_N (wn0, 0, 4 * q + 1, lane) * TROW + m] = v[q].y;
        smem[ACC_N (wn0, 0, 4 * q + 2, lane) * TROW + m] = v[q].z;
        smem[ACC_N (wn0, 0, 4 * q + 3, lane) * TROW + m] = v[q].w;
    }
    __syncthreads ();
}

// ---------------------------------------------------------------------------------------------
// Bandwidth tiles: 128-bit accesses, a tile = tile_n whole columns.
// ---------------------------------------------------------------------------------------------
template <int COH>
__device__ __forceinline__ void tile_residual (const aspen_hip_layer_t &L, uint32_t tn)
{
    const uint32_t n0 = tn * L.tile_n, n1 = min (n0 + L.tile_n, L.N), M4 = L.ld >> 2;
    const uint32_t total = (n1 - n0) * M4;
    ActView<COH> p0, p1, out;
    p0.init (L.in0, L.N, L.ld0); p1.init (L.in1, L.N, L.ld1); out.init (L.out, L.N, L.ld);
    // two pieces per thread and step: four loads in flight before the first store (the second piece of a thread's last
    // step may lie past the end: it is then fetched from the last piece's address and not stored)
    for (uint32_t i0 = tile_thread (); i0 < total; i0 += 2 * WG_THREADS)
    {
        float4 a[2], b[2];
        uint32_t dst[2];
        #pragma unroll
        for (int u = 0; u < 2; u++)
        {
            const uint32_t i = min (i0 + u * WG_THREADS, total - 1), c = i / M4, m = (i - c * M4) * 4, n = n0 + c;
            a[u] = p0.ld4 (n * L.ld0 + m); b[u] = p1.ld4 (n * L.ld1 + m);
            dst[u] = n * L.ld + m;
        }
        #pragma unroll
        for (int u = 0; u < 2; u++)
        {
            if (u && i0 + WG_THREADS >= total) break;
            a[u].x += b[u].x; a[u].y += b[u].y; a[u].z += b[u].z; a[u].w += b[u].w;
            out.st4 (dst[u], act4 (a[u], L.act));
        }
    }
}

// One thread = four channels of TWO neighbouring output positions.  Where both lie in the same output row their
// windows overlap by KW - stride input columns (a 3x3 / stride-2 pool fetches every input 2.25 times when each
// output loads its own window): the union of the two windows is fetched once, 15 instead of 18 loads for 3x3 / 2.
template <bool IS_MAX, int COH>
__device__ __forceinline__ void tile_pool (const aspen_hip_layer_t &L, uint32_t tn, uint32_t tm)
{
    // rows [r0, r1) of the tile; the last row tile also covers the padding rows up to the stride
    const uint32_t r0 = tm * L.tile_m, r1 = tm + 1 == L.tiles_m ? L.ld : r0 + L.tile_m;
    const uint32_t n0 = tn * L.tile_n, n1 = min (n0 + L.tile_n, L.N), M4 = (r1 - r0) >> 2;
    // pairing pays only where neighbouring windows overlap; elsewhere a thread keeps to one position
    const uint32_t per_thread = (L.KW > L.stride && L.OW > 1) ? 2u : 1u;
    const uint32_t pairs = (n1 - n0 + per_thread - 1) / per_thread, total = pairs * M4, ohw = L.OH * L.OW;
    const float inv = 1.0f / (float)(L.KH * L.KW);
    ActView<COH> in, out;
    in.init (L.in0, (L.N / ohw) * L.IH * L.IW, L.ld0); out.init (L.out, L.N, L.ld);
    const float4 start = IS_MAX ? make_float4 (-INFINITY, -INFINITY, -INFINITY, -INFINITY) : make_float4 (0.f, 0.f, 0.f, 0.f);
    auto combine = [] (float4 &r, const float4 &x)
    {
        if (IS_MAX) { r.x = r.x >= x.x ? r.x : x.x; r.y = r.y >= x.y ? r.y : x.y; r.z = r.z >= x.z ? r.z : x.z; r.w = r.w >= x.w ? r.w : x.w; }
        else { r.x += x.x; r.y += x.y; r.z += x.z; r.w += x.w; }
    };
    auto finish = [&] (float4 r, uint32_t n, uint32_t m)
    {
        if (!IS_MAX) { r.x *= inv; r.y *= inv; r.z *= inv; r.w *= inv; }
        r = act4 (r, L.act);
        // keep the zero padding rows [M, ld) intact
        if (m + 4 > L.M) { if (m + 0 >= L.M) r.x = 0.f; if (m + 1 >= L.M) r.y = 0.f; if (m + 2 >= L.M) r.z = 0.f; if (m + 3 >= L.M) r.w = 0.f; }
        out.st4 (n * L.ld + m, r);
    };
    if (per_thread == 1 && L.KH * L.KW >= 32)
    {
        // a wide window (global average pooling, 7x7 = 49 positions): eight neighbouring lanes share a piece, each
        // requests every eighth position of the window (all of its up to eight at once), and the eight partial results
        // meet through lane exchanges: one trip to memory per piece instead of one per window row.  (Sums are
        // formed in a different order than row by row: equal up to rounding.)
        const uint32_t sub = tile_thread () & 7u, P = L.KH * L.KW;
        for (uint32_t i0 = tile_thread () >> 3; i0 < (total + WG_THREADS / 8 - 1) / (WG_THREADS / 8) * (WG_THREADS / 8); i0 += WG_THREADS / 8)
        {
            // (every lane of a wavefront takes part in the exchanges: a group past the end works on the last piece and stores nothing)
            const uint32_t i = min (i0, total - 1);
            const uint32_t c = i / M4, m = r0 + (i - c * M4) * 4, n = n0 + c;
            const uint32_t b = n / ohw, rem = n - b * ohw, oh = rem / L.OW, ow = rem - oh * L.OW;
            const int ih0 = (int)(oh * L.stride) - (int)L.pad, iw0 = (int)(ow * L.stride) - (int)L.pad;
            float4 r = start;
            for (uint32_t p0 = 0; p0 < P; p0 += 64)
            {
                float4 x[8];
                #pragma unroll
                for (uint32_t q = 0; q < 8; q++)
                {
                    const uint32_t pos = min (p0 + sub + 8 * q, P - 1), kh = pos / L.KW, kw = pos - kh * L.KW;
                    const uint32_t ihc = (uint32_t)min (max (ih0 + (int)kh, 0), (int)L.IH - 1), iwc = (uint32_t)min (max (iw0 + (int)kw, 0), (int)L.IW - 1);
                    x[q] = in.ld4 (((b * L.IH + ihc) * L.IW + iwc) * L.ld0 + m);
                }
                #pragma unroll
                for (uint32_t q = 0; q < 8; q++)
                {
                    const uint32_t pos = p0 + sub + 8 * q, kh = pos / L.KW, kw = pos - kh * L.KW;
                    if (pos < P && (uint32_t)(ih0 + (int)kh) < L.IH && (uint32_t)(iw0 + (int)kw) < L.IW) combine (r, x[q]);
                }
            }
            #pragma unroll
            for (int o = 1; o < 8; o <<= 1)
            {
                float4 y;
                y.x = __shfl_xor (r.x, o, 64); y.y = __shfl_xor (r.y, o, 64); y.z = __shfl_xor (r.z, o, 64); y.w = __shfl_xor (r.w, o, 64);
                combine (r, y);
            }
            if (sub == 0 && i0 < total) finish (r, n, m);
        }
        return;
    }
    if (per_thread == 1 && L.KH == 2 && L.KW == 2)
    {
        // the 2x2 window of the VGG / Darknet pools: a thread requests the four inputs of two of its pieces together (clamped
        // to the image where padding puts them outside, and then not used); combined in the order of the general loop below
        for (uint32_t i0 = tile_thread (); i0 < total; i0 += 2 * WG_THREADS)
        {
            float4 x[2][4];
            uint32_t nn[2], mm[2];
            int ih0[2], iw0[2];
            #pragma unroll
            for (int u = 0; u < 2; u++)
            {
                const uint32_t i = min (i0 + u * WG_THREADS, total - 1);
                const uint32_t c = i / M4, m = r0 + (i - c * M4) * 4, n = n0 + c;
                const uint32_t b = n / ohw, rem = n - b * ohw, oh = rem / L.OW, ow = rem - oh * L.OW;
                nn[u] = n; mm[u] = m;
                ih0[u] = (int)(oh * L.stride) - (int)L.pad; iw0[u] = (int)(ow * L.stride) - (int)L.pad;
                #pragma unroll
                for (int q = 0; q < 4; q++)
                {
                    const uint32_t ihc = (uint32_t)min (max (ih0[u] + (q >> 1), 0), (int)L.IH - 1), iwc = (uint32_t)min (max (iw0[u] + (q & 1), 0), (int)L.IW - 1);
                    x[u][q] = in.ld4 (((b * L.IH + ihc) * L.IW + iwc) * L.ld0 + m);
                }
            }
            #pragma unroll
            for (int u = 0; u < 2; u++)
            {
                if (u && i0 + WG_THREADS >= total) break;
                float4 r = start;
                #pragma unroll
                for (int q = 0; q < 4; q++)
                    if ((uint32_t)(ih0[u] + (q >> 1)) < L.IH && (uint32_t)(iw0[u] + (q & 1)) < L.IW) combine (r, x[u][q]);
                finish (r, nn[u], mm[u]);
            }
        }
        return;
    }
    for (uint32_t i = tile_thread (); i < total; i += WG_THREADS)
    {
        const uint32_t c = i / M4, m = r0 + (i - c * M4) * 4, n = n0 + per_thread * c;
        const uint32_t b = n / ohw, rem = n - b * ohw, oh = rem / L.OW, ow = rem - oh * L.OW;
        const bool second = per_thread == 2 && n + 1 < n1, same_row = second && ow + 1 < L.OW;
        // windows of the two positions as one span of input columns when they share a row, else one window each
        const uint32_t span = same_row ? L.KW + L.stride : L.KW;
        for (uint32_t which = 0; which < (second && !same_row ? 2u : 1u); which++)
        {
            const uint32_t nn = n + which;
            uint32_t bb = b, hh = oh, ww = ow;
            if (which) { ww = ow + 1; if (ww == L.OW) { ww = 0; if (++hh == L.OH) { hh = 0; ++bb; } } }
            float4 ra = start, rb = start;
            if (same_row && L.KH == 3 && L.KW == 3 && L.stride == 2)
            {
                // two neighbouring 3x3 / stride-2 windows (the ResNet stem's pool): all fifteen inputs are requested
                // together; clamped where padding puts them outside the image, and then not used
                const int ih0 = (int)(hh * L.stride) - (int)L.pad, iw0 = (int)(ww * L.stride) - (int)L.pad;
                float4 x[3][5];
                #pragma unroll
                for (int kh = 0; kh < 3; kh++)
                {
                    const uint32_t row = (bb * L.IH + (uint32_t)min (max (ih0 + kh, 0), (int)L.IH - 1)) * L.IW;
                    #pragma unroll
                    for (int q = 0; q < 5; q++) x[kh][q] = in.ld4 ((row + (uint32_t)min (max (iw0 + q, 0), (int)L.IW - 1)) * L.ld0 + m);
                }
                #pragma unroll
                for (int kh = 0; kh < 3; kh++)
                {
                    if ((uint32_t)(ih0 + kh) >= L.IH) continue;
                    #pragma unroll
                    for (int q = 0; q < 5; q++)
                    {
                        if ((uint32_t)(iw0 + q) >= L.IW) continue;
                        if (q < 3) combine (ra, x[kh][q]);
                        if (q >= 2) combine (rb, x[kh][q]);
                    }
                }
                finish (ra, nn, m);
                finish (rb, nn + 1, m);
                continue;
            }
            for (uint32_t kh = 0; kh < L.KH; kh++)
            {
                const int ih = (int)(hh * L.stride + kh) - (int)L.pad;
                if ((uint32_t)ih >= L.IH) continue;
                if (span > 4)
                {
                    // a wide window (global average pooling): eight positions of the row are requested at once, so that
                    // their memory latencies overlap; positions outside the window or the image are fetched from a
                    // clamped, valid address and not used.  Same order of additions as the plain loop below.
                    const uint32_t row = (bb * L.IH + ih) * L.IW;
                    for (uint32_t kw0 = 0; kw0 < span; kw0 += 8)
                    {
                        float4 x[8];
                        #pragma unroll
                        for (uint32_t q = 0; q < 8; q++)
                        {
                            const int iw = (int)(ww * L.stride + kw0 + q) - (int)L.pad;
                            const uint32_t iwc = (uint32_t)min (max (iw, 0), (int)L.IW - 1);
                            x[q] = in.ld4 ((row + iwc) * L.ld0 + m);
                        }
                        #pragma unroll
                        for (uint32_t q = 0; q < 8; q++)
                        {
                            const uint32_t kw = kw0 + q;
                            const int iw = (int)(ww * L.stride + kw) - (int)L.pad;
                            if (kw >= span || (uint32_t)iw >= L.IW) continue;
                            if (kw < L.KW) combine (ra, x[q]);
                            if (same_row && kw >= L.stride) combine (rb, x[q]);
                        }
                    }
                    continue;
                }
                for (uint32_t kw = 0; kw < span; kw++)
                {
                    const int iw = (int)(ww * L.stride + kw) - (int)L.pad;
                    if ((uint32_t)iw >= L.IW) continue;
                    const float4 x = in.ld4 (((bb * L.IH + ih) * L.IW + iw) * L.ld0 + m);
                    if (kw < L.KW) combine (ra, x);
                    if (same_row && kw >= L.stride) combine (rb, x);
                }
            }
            finish (ra, nn, m);
            if (same_row) finish (rb, nn + 1, m);
        }
    }
}

// YOLO box decode (reference tiled_yolo, src/tiled_kernels.c:675-708).  Output column = (batch, anchor,
// cell); rows = classes + 5 read from channels [anchor * M, anchor * M + M) of input column (batch, cell).
// L.weight holds the three anchor boxes (w0, h0, w1, h1, w2, h2).
// One thread per four consecutive rows of a column: the output piece is one aligned 16-byte store; the four
// inputs start at channel anchor * M, which is not 16-byte aligned in general, and are fetched as four
// dwords (neighbouring lanes read neighbouring dwords, so the wave still covers whole cache lines).
template <int COH>
__device__ __forceinline__ void tile_yolo (const aspen_hip_layer_t &L, uint32_t tn)
{
    const uint32_t n0 = tn * L.tile_n, n1 = min (n0 + L.tile_n, L.N);
    const uint32_t cells = L.IH * L.IW, A = L.IC / L.M, pieces = (L.M + 3) >> 2, total = (n1 - n0) * pieces;
    const float stride = (float)L.stride;
    ActView<COH> in, out;
    in.init (L.in0, (L.N / (cells * A)) * cells, L.ld0); out.init (L.out, L.N, L.ld);
    for (uint32_t i = tile_thread (); i < total; i += WG_THREADS)
    {
        const uint32_t c = i / pieces, j = (i - c * pieces) * 4, n = n0 + c;
        const uint32_t seg = n / cells, b = seg / A, a = seg - b * A, cell = n - seg * cells;
        const uint32_t src = (b * cells + cell) * L.ld0 + a * L.M + j, left = L.M - j;
        float x[4], r[4];
        #pragma unroll
        for (uint32_t k = 0; k < 4; k++) x[k] = k < left ? in.ld1 (src + k) : 0.f;
        #pragma unroll
        for (uint32_t k = 0; k < 4; k++) r[k] = 1.0f / (1.0f + expf (-x[k]));
        if (j == 0)
        {
            const uint32_t h = cell / L.IW, w = cell - h * L.IW;
            r[0] = (r[0] + (float)w) * stride;
            r[1] = (r[1] + (float)h) * stride;
            r[2] = expf (x[2]) * gld1 (L.weight + 2 * a);
            r[3] = expf (x[3]) * gld1 (L.weight + 2 * a + 1);
        }
        const uint32_t dst = n * L.ld + j;
        if (left >= 4) out.st4 (dst, make_float4 (r[0], r[1], r[2], r[3]));
        else { out.st1 (dst, r[0]); if (left > 1) out.st1 (dst + 1, r[1]); if (left > 2) out.st1 (dst + 2, r[2]); }
    }
}

// Nearest-neighbour upsampling of the first parent by `stride`, concatenated along the channels with
// the second parent (reference tiled_append, src/tiled_kernels.c:710-741).  IC = channels of the first parent.
// Both parts of an output column are contiguous copies: 16 bytes per thread when the channel counts are
// multiples of four (then every piece is aligned and lies within one part), one float per thread otherwise.
template <int COH>
__device__ __forceinline__ void tile_append (const aspen_hip_layer_t &L, uint32_t tn)
{
    const uint32_t n0 = tn * L.tile_n, n1 = min (n0 + L.tile_n, L.N);
    const uint32_t ohw = L.OH * L.OW, iw = L.OW / L.stride, ih = L.OH / L.stride;
    ActView<COH> p0, p1, out;
    p0.init (L.in0, (L.N / ohw) * ih * iw, L.ld0); p1.init (L.in1, L.N, L.ld1); out.init (L.out, L.N, L.ld);
    if (((L.IC | L.M) & 3u) == 0)
    {
        const uint32_t M4 = L.M >> 2, total = (n1 - n0) * M4;
        // four pieces per thread and step, all requested before the first store (pieces past the end: fetched from the
        // last piece's address and not stored)
        for (uint32_t i0 = tile_thread (); i0 < total; i0 += 4 * WG_THREADS)
        {
            float4 v[4];
            uint32_t dst[4];
            #pragma unroll
            for (int u = 0; u < 4; u++)
            {
                const uint32_t i = min (i0 + u * WG_THREADS, total - 1), c = i / M4, m = (i - c * M4) * 4, n = n0 + c;
                const uint32_t b = n / ohw, rem = n - b * ohw, oh = rem / L.OW, ow = rem - oh * L.OW;
                v[u] = m < L.IC ? p0.ld4 (((b * ih + oh / L.stride) * iw + ow / L.stride) * L.ld0 + m)
                                : p1.ld4 (n * L.ld1 + (m - L.IC));
                dst[u] = n * L.ld + m;
            }
            #pragma unroll
            for (int u = 0; u < 4; u++)
                if (i0 + u * WG_THREADS < total) out.st4 (dst[u], v[u]);
        }
        return;
    }
    const uint32_t total = (n1 - n0) * L.M;
    for (uint32_t i = tile_thread (); i < total; i += WG_THREADS)
    {
        const uint32_t c = i / L.M, m = i - c * L.M, n = n0 + c;
        const uint32_t b = n / ohw, rem = n - b * ohw, oh = rem / L.OW, ow = rem - oh * L.OW;
        const float v = m < L.IC ? p0.ld1 (((b * ih + oh / L.stride) * iw + ow / L.stride) * L.ld0 + m)
                                 : p1.ld1 (n * L.ld1 + (m - L.IC));
        out.st1 (n * L.ld + m, v);
    }
}

__device__ __forceinline__ float wave_sum (float v)
{
    #pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor (v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max (float v)
{
    #pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf (v, __shfl_xor (v, o, 64));
    return v;
}

// One wavefront per column, the column kept in registers between the two passes (16 bytes x COLUMN_CACHE per
// lane: columns of up to 64 * 4 * COLUMN_CACHE floats are read once; longer ones are read again).
#define COLUMN_CACHE 4

// mean and E[x^2] in one pass, eps 1e-6f (reference tiled_layernorm, src/tiled_kernels.c:743-783)
template <int COH>
__device__ __forceinline__ void tile_layernorm (const aspen_hip_layer_t &L, uint32_t tn)
{
    const uint32_t n0 = tn * L.tile_n, n1 = min (n0 + L.tile_n, L.N);
    const uint32_t lane = tile_thread () & 63, wave = tile_thread () >> 6, M4 = L.M >> 2;
    ActView<COH> in, out;
    in.init (L.in0, L.N, L.ld0); out.init (L.out, L.N, L.ld);
    // this lane's scale and shift are the same for every column
    float4 g[COLUMN_CACHE], b[COLUMN_CACHE];
    #pragma unroll
    for (uint32_t k = 0; k < COLUMN_CACHE; k++)
    {
        const uint32_t m = lane + 64 * k;
        g[k] = m < M4 ? gld4 (L.weight + m * 4) : make_float4 (0.f, 0.f, 0.f, 0.f);
        b[k] = (m < M4 && L.bias) ? gld4 (L.bias + m * 4) : make_float4 (0.f, 0.f, 0.f, 0.f);
    }
    for (uint32_t n = n0 + wave; n < n1; n += WG_THREADS / 64)
    {
        const uint32_t x = n * L.ld0, o = n * L.ld;
        float4 v[COLUMN_CACHE];
        #pragma unroll
        for (uint32_t k = 0; k < COLUMN_CACHE; k++)
            v[k] = lane + 64 * k < M4 ? in.ld4 (x + (lane + 64 * k) * 4) : make_float4 (0.f, 0.f, 0.f, 0.f);
        float s = 0.f, q = 0.f;
        #pragma unroll
        for (uint32_t k = 0; k < COLUMN_CACHE; k++)
        {
            s += v[k].x + v[k].y + v[k].z + v[k].w;
            q += v[k].x * v[k].x + v[k].y * v[k].y + v[k].z * v[k].z + v[k].w * v[k].w;
        }
        for (uint32_t m = lane + 64 * COLUMN_CACHE; m < M4; m += 64)
        {
            const float4 w = in.ld4 (x + m * 4);
            s += w.x + w.y + w.z + w.w;
            q += w.x * w.x + w.y * w.y + w.z * w.z + w.w * w.w;
        }
        for (uint32_t m = M4 * 4 + lane; m < L.M; m += 64) { const float w = in.ld1 (x + m); s += w; q += w * w; }
        s = wave_sum (s); q = wave_sum (q);
        const float mean = s / (float)L.M;
        float var = q / (float)L.M - mean * mean;
        const float rstd = 1.0f / sqrtf (var + 1e-6f);
        #pragma unroll
        for (uint32_t k = 0; k < COLUMN_CACHE; k++)
            if (lane + 64 * k < M4)
            {
                float4 r;
                r.x = (v[k].x - mean) * rstd * g[k].x; r.y = (v[k].y - mean) * rstd * g[k].y;
                r.z = (v[k].z - mean) * rstd * g[k].z; r.w = (v[k].w - mean) * rstd * g[k].w;
                if (L.bias) { r.x += b[k].x; r.y += b[k].y; r.z += b[k].z; r.w += b[k].w; }
                out.st4 (o + (lane + 64 * k) * 4, r);
            }
        for (uint32_t m = lane + 64 * COLUMN_CACHE; m < M4; m += 64)
        {
            const float4 w = in.ld4 (x + m * 4), gg = gld4 (L.weight + m * 4);
            float4 r;
            r.x = (w.x - mean) * rstd * gg.x; r.y = (w.y - mean) * rstd * gg.y;
            r.z = (w.z - mean) * rstd * gg.z; r.w = (w.w - mean) * rstd * gg.w;
            if (L.bias) { const float4 bb = gld4 (L.bias + m * 4); r.x += bb.x; r.y += bb.y; r.z += bb.z; r.w += bb.w; }
            out.st4 (o + m * 4, r);
        }
        for (uint32_t m = M4 * 4 + lane; m < L.M; m += 64)
            out.st1 (o + m, (in.ld1 (x + m) - mean) * rstd * gld1 (L.weight + m) + (L.bias ? gld1 (L.bias + m) : 0.f));
    }
}

// max-subtracted softmax over the rows of a column (reference tiled_softmax, src/tiled_kernels.c:640-673)
template <int COH>
__device__ __forceinline__ void tile_softmax (const aspen_hip_layer_t &L, uint32_t tn)
{
    const uint32_t n0 = tn * L.tile_n, n1 = min (n0 + L.tile_n, L.N);
    const uint32_t lane = tile_thread () & 63, wave = tile_thread () >> 6, M4 = L.M >> 2;
    ActView<COH> in, out;
    in.init (L.in0, L.N, L.ld0); out.init (L.out, L.N, L.ld);
    for (uint32_t n = n0 + wave; n < n1; n += WG_THREADS / 64)
    {
        const uint32_t x = n * L.ld0, o = n * L.ld;
        const float4 low = make_float4 (-INFINITY, -INFINITY, -INFINITY, -INFINITY);
        float4 v[COLUMN_CACHE];
        #pragma unroll
        for (uint32_t k = 0; k < COLUMN_CACHE; k++) v[k] = lane + 64 * k < M4 ? in.ld4 (x + (lane + 64 * k) * 4) : low;
        float mx = -INFINITY;
        #pragma unroll
        for (uint32_t k = 0; k < COLUMN_CACHE; k++) mx = fmaxf (mx, fmaxf (fmaxf (v[k].x, v[k].y), fmaxf (v[k].z, v[k].w)));
        for (uint32_t m = (lane + 64 * COLUMN_CACHE) * 4; m < M4 * 4; m += 256) { const float4 w = in.ld4 (x + m); mx = fmaxf (mx, fmaxf (fmaxf (w.x, w.y), fmaxf (w.z, w.w))); }
        for (uint32_t m = M4 * 4 + lane; m < L.M; m += 64) mx = fmaxf (mx, in.ld1 (x + m));
        mx = wave_max (mx);
        // the exponentials of the cached part are computed once; exp (-inf) = 0 for the lanes past the column
        float s = 0.f;
        #pragma unroll
        for (uint32_t k = 0; k < COLUMN_CACHE; k++)
        {
            v[k] = make_float4 (expf (v[k].x - mx), expf (v[k].y - mx), expf (v[k].z - mx), expf (v[k].w - mx));
            s += v[k].x + v[k].y + v[k].z + v[k].w;
        }
        for (uint32_t m = (lane + 64 * COLUMN_CACHE) * 4; m < M4 * 4; m += 256)
        { const float4 w = in.ld4 (x + m); s += expf (w.x - mx) + expf (w.y - mx) + expf (w.z - mx) + expf (w.w - mx); }
        for (uint32_t m = M4 * 4 + lane; m < L.M; m += 64) s += expf (in.ld1 (x + m) - mx);
        s = wave_sum (s);
        #pragma unroll
        for (uint32_t k = 0; k < COLUMN_CACHE; k++)
            if (lane + 64 * k < M4) out.st4 (o + (lane + 64 * k) * 4, make_float4 (v[k].x / s, v[k].y / s, v[k].z / s, v[k].w / s));
        for (uint32_t m = (lane + 64 * COLUMN_CACHE) * 4; m < M4 * 4; m += 256)
        { const float4 w = in.ld4 (x + m); out.st4 (o + m, make_float4 (expf (w.x - mx) / s, expf (w.y - mx) / s, expf (w.z - mx) / s, expf (w.w - mx) / s)); }
        for (uint32_t m = M4 * 4 + lane; m < L.M; m += 64) out.st1 (o + m, expf (in.ld1 (x + m) - mx) / s);
    }
}

// ---------------------------------------------------------------------------------------------
// Attention tiles.
// K tile: one (batch, head) x KATTN_BN queries x all keys.  (32 queries, four wavefronts side by side along the keys: a
// tile works through its key blocks one after the other, and with 64 queries a long sequence has few tiles that each
// take long; GPT-2 at 512 tokens 3.95 -> 3.83 ms, one launch per layer 4.43 -> 4.17; BERT at 128 tokens 2.24 -> 2.26
// and 2.40 -> 2.32.  Both sizes in one kernel, chosen per layer, cost BERT 5 % through the register allocation.)  scores = K.Q on the matrix cores, 128 keys at
// a time; causal mask (-1e10 before the 1/sqrt(hd) scale), exp without max subtraction; every block's
// exponentials are stored (staged through LDS for 16-byte stores) while the queries' sums accumulate,
// then a sweep over the tile's own output divides by the sums.  Key blocks the causal mask zeroes for
// every query of the tile are not computed at all.
// in0 = Query matrix, in1 = Key matrix (reference cfg: parent = Query, from = Key).
// ---------------------------------------------------------------------------------------------
template <int COH>
__device__ __forceinline__ void tile_k_attention (const aspen_hip_layer_t &L, uint32_t tn, float *smem)
{
    constexpr int BM = 128, BN = KATTN_BN, WM = BN == 32 ? 4 : 2, WN = BN == 32 ? 1 : 2, TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr int TROW = BM + 8;            // staging row of one query: (4 * TROW) % 64 == 32, see the contraction epilogue
    static_assert (BN * TROW <= GEMM_SMEM_FLOATS, "probability staging fits the GEMM stage");
    __shared__ float rowsum[BN];
    const uint32_t tid = tile_thread (), lane = tid & 63, wave = tid >> 6;
    const uint32_t S = L.seq, qtiles = (S + BN - 1) / BN;
    const uint32_t bh = tn / qtiles, q0 = (tn - bh * qtiles) * BN;
    const uint32_t b = bh / L.heads, h = bh - b * L.heads;
    const uint32_t wm0 = (wave % WM) * (BM / WM), wn0 = (wave / WM) * (BN / WN);
    ActView<COH> Q, Kmat, out;
    Q.init (L.in0, L.N / L.heads, L.ld0); Kmat.init (L.in1, L.N / L.heads, L.ld1); out.init (L.out, L.N, L.ld);
    const uint32_t obase = bh * S * L.ld;                // column (b*H + h)*S + q, rows = keys
    const float scale = 1.0f / sqrtf ((float)L.hd);
    const uint32_t nq = min ((uint32_t)BN, S - q0);
    // with the causal mask every key beyond the tile's last query is masked for all of its queries:
    // exp (-1e10 * scale) is exactly 0, so those key blocks add nothing to the sums and are written as zeros
    const uint32_t kend = L.masked ? min (S, q0 + (uint32_t)BN) : S;
    const int kiters = (int)(L.hd / GEMM_BK);
    if (tid < BN) rowsum[tid] = 0.f;                     // ordered before the atomics below by the barriers of gemm_core

    // The scores are computed once: every key block's exponentials are stored unnormalised while the queries'
    // sums accumulate, and a second sweep over the tile's own output (still in this XCD's L2) divides by them.
    auto scores = [&] (uint32_t k0, floatx16 (&acc)[TN][TM])
    {
        ActRowLoader<BM, COH> al; al.init (Kmat, b * S + k0, b * S + S - 1, L.ld1, h * L.hd, tid);
        ActRowLoader<BN, COH> bl; bl.init (Q, b * S + q0, b * S + S - 1, L.ld0, h * L.hd, tid);
        gemm_core<BM, BN, WM, WN, 1> (al, bl, 0, kiters, smem, acc);
    };
    // exponential of one score; reference order of operations: mask with -1e10, scale, exp, no max subtraction.
    // The hardware exponential (2^(x log2 e), about 1e-6 relative for scores of a few units against libm's expf, two
    // orders inside the parity tolerance; exactly 0 for the masked -1e10): the tile is bound by this arithmetic,
    // 32 exponentials per lane and key block, and expf costs five times the instructions.
    auto weight = [&] (float sc, uint32_t key, uint32_t q) -> float
    {
        if (L.masked && key > q) sc = -1e10f;
        return (key < S && q < S) ? __expf (sc * scale) : 0.f;
    };

    float part[TN][16];
    #pragma unroll
    for (int i = 0; i < TN; i++)
        #pragma unroll
        for (int v = 0; v < 16; v++) part[i][v] = 0.f;
    constexpr uint32_t C4 = BM / 4, STEP = WG_THREADS / C4;
    const uint32_t c = (tid % C4) * 4;
    for (uint32_t k0 = 0; k0 < kend; k0 += BM)
    {
        floatx16 acc[TN][TM];
        scores (k0, acc);                                // ends with a barrier: the stage is free
        #pragma unroll
        for (int i = 0; i < TN; i++)
            #pragma unroll
            for (int v = 0; v < 16; v++)
            {
                const uint32_t ql = ACC_N (wn0, i, v, lane);
                #pragma unroll
                for (int j = 0; j < TM; j++)
                {
                    const float e = weight (acc[i][j][v], k0 + wm0 + 32 * j + (lane & 31), q0 + ql);
                    part[i][v] += e;
                    smem[ql * TROW + wm0 + 32 * j + (lane & 31)] = e;
                }
            }
        __syncthreads ();
        for (uint32_t r = tid / C4; r < nq; r += STEP)
        {
            const float4 p = ld4 (smem + r * TROW + c);
            const uint32_t key = k0 + c, o = obase + (q0 + r) * L.ld + key;
            if (key + 4 <= S) out.st4 (o, p);
            else if (key < S) { out.st1 (o, p.x); if (key + 1 < S) out.st1 (o + 1, p.y); if (key + 2 < S) out.st1 (o + 2, p.z); }
        }
        __syncthreads ();                                // the next block's operands overwrite the stage
    }
    // row sums: 32 lanes of a half-wave hold 32 different keys of the same query
    #pragma unroll
    for (int i = 0; i < TN; i++)
        #pragma unroll
        for (int v = 0; v < 16; v++)
        {
            float t = part[i][v];
            #pragma unroll
            for (int o = 16; o > 0; o >>= 1) t += __shfl_xor (t, o, 64);
            if ((lane & 31) == 0) atomicAdd (&rowsum[ACC_N (wn0, i, v, lane)], t);
        }
    asm volatile ("s_waitcnt vmcnt(0)" ::: "memory");   // this workgroup's own stores, read back below
    __syncthreads ();
    // second sweep over the tile's own output: divide by the sums
    const uint32_t kcov = min (S, (kend + BM - 1) / BM * BM);
    for (uint32_t k0 = 0; k0 < kcov; k0 += BM)
        for (uint32_t r = tid / C4; r < nq; r += STEP)
        {
            const uint32_t key = k0 + c, o = obase + (q0 + r) * L.ld + key;
            const float inv = 1.0f / rowsum[r];             // one division per piece, then products (within an ulp of the quotients)
            if (key + 4 <= S)
            {
                float4 p = out.ld4 (o);
                p.x *= inv; p.y *= inv; p.z *= inv; p.w *= inv;
                out.st4 (o, p);
            }
            else
                for (uint32_t e = key; e < S; e++) out.st1 (o + e - key, out.ld1 (o + e - key) * inv);
        }
    // key blocks that are masked for every query of the tile
    for (uint32_t k0 = (kend + BM - 1) / BM * BM; k0 < S; k0 += BM)
        for (uint32_t r = tid / C4; r < nq; r += STEP)
        {
            const uint32_t key = k0 + c, o = obase + (q0 + r) * L.ld + key;
            if (key + 4 <= S) out.st4 (o, make_float4 (0.f, 0.f, 0.f, 0.f));
            else if (key < S) { out.st1 (o, 0.f); if (key + 1 < S) out.st1 (o + 1, 0.f); if (key + 2 < S) out.st1 (o + 2, 0.f); }
        }
    __syncthreads ();
}

// V tile: one (batch, head-slice of <= 64 channels) x VATTN_BN queries:
// out[b*S + q][h*hd + j] = sum_s P[(b*H + h)*S + q][s] * V[b*S + s][h*hd + j].
// in0 = probabilities (K-attention output), in1 = Value matrix.
template <int COH>
__device__ __forceinline__ void tile_v_attention (const aspen_hip_layer_t &L, uint32_t tn, uint32_t tm, float *smem)
{
    constexpr int BM = 64, BN = VATTN_BN, WM = 2, WN = 2, TM = 1, TN = BN / WN / 32;
    const uint32_t tid = tile_thread (), lane = tid & 63, wave = tid >> 6;
    const uint32_t S = L.seq, qtiles = (S + BN - 1) / BN;
    const uint32_t b = tn / qtiles, q0 = (tn - b * qtiles) * BN;
    const uint32_t m0 = tm * L.tile_m, h = m0 / L.hd;
    const uint32_t wm0 = (wave % WM) * (BM / WM), wn0 = (wave / WM) * (BN / WN);
    ActView<COH> P, V, out;
    P.init (L.in0, L.N * L.heads, L.ld0); V.init (L.in1, L.N, L.ld1); out.init (L.out, L.N, L.ld);
    const uint32_t prow = (b * L.heads + h) * S;
    floatx16 acc[TN][TM];
    TransLoader64<COH> al; al.init (V, b * S * L.ld1 + m0, L.ld1, L.tile_m, S, tid);
    ActRowLoader<BN, COH> bl; bl.init (P, prow + q0, prow + S - 1, L.ld0, 0, tid);   // P's stride is a multiple of 32 with zero padding
    gemm_core<BM, BN, WM, WN, 1> (al, bl, 0, (int)((S + GEMM_BK - 1) / GEMM_BK), smem, acc);
    const uint32_t mm = wm0 + (lane & 31);
    if (mm < L.tile_m)
        #pragma unroll
        for (int i = 0; i < TN; i++)
            #pragma unroll
            for (int v = 0; v < 16; v++)
            {
                const uint32_t q = q0 + ACC_N (wn0, i, v, lane);
                if (q < S) out.st1 ((b * S + q) * L.ld + m0 + mm, acc[i][0][v]);
            }
}

// Fused attention tile: one (batch, head) x VATTN_BN queries, scores and weighted values in one pass, the S x S
// probability matrix never leaves the chip (reference: tiled_k_attention followed by tiled_v_attention,
// src/tiled_kernels.c:784-1037, which round-trip it through memory).  Per block of 64 keys:
//   e[q][key] = exp (scale * (key > q && masked ? -1e10 : K[key] . Q[q]))      (the reference's order of operations,
//                                                                               no max subtraction)
//   rowsum[q] += sum_key e[q][key];   O[q][ch] += sum_key e[q][key] * V[key][ch]
// and at the end O[q][ch] / rowsum[q].  The reference divides the probabilities first and multiplies then; dividing
// the sum of products instead differs by rounding only (1e-7 relative).  The exponentials of a key block go to LDS in
// the layout of an activation operand (row = query, K axis = key), the transposed values are staged next to them.
// in0 = Query, in1 = Key, fuse_in = Value (stride fuse_ld_in); one head of at most 64 channels per tile.
// Used when nothing but the V-attention layer reads the probabilities and their matrix need not be kept.
// ---------------------------------------------------------------------------------------------
template <int COH>
__device__ __forceinline__ void tile_fused_attention (const aspen_hip_layer_t &L, uint32_t tn, uint32_t tm, float *smem)
{
    constexpr int BQ = VATTN_BN, BKEY = 64, EROW = BKEY + 4;
    static_assert (BQ == 64, "four wavefronts, one 32 x 32 block each");
    static_assert ((64 + BQ) * LDS_ROW + BQ * EROW <= GEMM_SMEM_FLOATS, "operand stage and exponentials fit the tile's LDS");
    __shared__ float qsum[BQ];
    const uint32_t tid = tile_thread (), lane = tid & 63, wave = tid >> 6;
    const uint32_t S = L.seq, qtiles = (S + BQ - 1) / BQ;
    const uint32_t b = tn / qtiles, q0 = (tn - b * qtiles) * BQ;
    const uint32_t h = tm, hd = L.hd;
    const uint32_t wm0 = (wave % 2) * 32, wn0 = (wave / 2) * 32;       // keys (phase 1) / channels (phase 2), queries
    ActView<COH> Q, Kmat, V, out;
    Q.init (L.in0, L.N, L.ld0); Kmat.init (L.in1, L.N, L.ld1); V.init (L.fuse_in, L.N, L.fuse_ld_in); out.init (L.out, L.N, L.ld);
    const float scale = 1.0f / sqrtf ((float)hd);
    const uint32_t kend = L.masked ? min (S, q0 + (uint32_t)BQ) : S;
    const int kiters = (int)(hd / GEMM_BK);
    float *ebuf = smem + (64 + BQ) * LDS_ROW;
    if (tid < BQ) qsum[tid] = 0.f;                       // ordered before the atomics below by the barriers of the K loops
    floatx16 oacc;
    float part[16];
    #pragma unroll
    for (int v = 0; v < 16; v++) { oacc[v] = 0.f; part[v] = 0.f; }
    for (uint32_t k0 = 0; k0 < kend; k0 += BKEY)
    {
        // the block's first 32 rows of V are requested before the scores are computed (they do not depend on them): one
        // trip to memory less on the path of a tile whose key blocks run one after the other
        TransLoader64<COH> vl;
        vl.init (V, (b * S + k0) * L.fuse_ld_in + h * hd, L.fuse_ld_in, hd, S - k0, tid);
        float4 vreg[2];
        vl.load (0, vreg);
        // scores of 64 keys x 64 queries: one 32 x 32 block per wavefront
        floatx16 sacc[1][1];
        {
            ActRowLoader<64, COH> al; al.init (Kmat, b * S + k0, b * S + S - 1, L.ld1, h * hd, tid);
            ActRowLoader<BQ, COH> bl; bl.init (Q, b * S + q0, b * S + S - 1, L.ld0, h * hd, tid);
            gemm_core_single_block<1> (al, bl, 0, kiters, smem, sacc);          // ends with a barrier: the stage is free
        }
        #pragma unroll
        for (int v = 0; v < 16; v++)
        {
            const uint32_t ql = ACC_N (wn0, 0, v, lane), key = k0 + wm0 + (lane & 31), q = q0 + ql;
            float sc = sacc[0][0][v];
            if (L.masked && key > q) sc = -1e10f;
            const float e = (key < S && q < S) ? __expf (sc * scale) : 0.f;
            part[v] += e;
            ebuf[ql * EROW + wm0 + (lane & 31)] = e;
        }
        // weighted values: O[q][ch] += e[q][key] V[key][ch], two slices of 32 keys; V is read transposed through the stage
        #pragma unroll
        for (int sl = 0; sl < BKEY / GEMM_BK; sl++)
        {
            vl.store (smem, vreg);
            if (sl + 1 < BKEY / GEMM_BK) vl.load (sl + 1, vreg);
            __syncthreads ();                            // the stage and (first slice) the exponentials are complete
            const float *af = smem + (wm0 + (lane & 31)) * LDS_ROW + (lane >> 5) * 4;
            const float *bf = ebuf + (wn0 + (lane & 31)) * EROW + sl * GEMM_BK + (lane >> 5) * 4;
            #pragma unroll
            for (int sub = 0; sub < 4; sub++)
            {
                const float4 a = ld4 (af + sub * 8), e4 = ld4 (bf + sub * 8);
                oacc = __builtin_amdgcn_mfma_f32_32x32x2f32 (e4.x, a.x, oacc, 0, 0, 0);
                oacc = __builtin_amdgcn_mfma_f32_32x32x2f32 (e4.y, a.y, oacc, 0, 0, 0);
                oacc = __builtin_amdgcn_mfma_f32_32x32x2f32 (e4.z, a.z, oacc, 0, 0, 0);
                oacc = __builtin_amdgcn_mfma_f32_32x32x2f32 (e4.w, a.w, oacc, 0, 0, 0);
            }
            __syncthreads ();                            // everyone has read the stage (and, last slice, the exponentials)
        }
    }
    // row sums: the 32 lanes of a half-wave hold 32 keys of the same query; two wavefronts share a query block
    #pragma unroll
    for (int v = 0; v < 16; v++)
    {
        float t = part[v];
        #pragma unroll
        for (int o = 16; o > 0; o >>= 1) t += __shfl_xor (t, o, 64);
        if ((lane & 31) == 0) atomicAdd (&qsum[ACC_N (wn0, 0, v, lane)], t);
    }
    __syncthreads ();
    const uint32_t ch = wm0 + (lane & 31);
    if (ch < hd)
        #pragma unroll
        for (int v = 0; v < 16; v++)
        {
            const uint32_t ql = ACC_N (wn0, 0, v, lane), q = q0 + ql;
            if (q < S) out.st1 ((b * S + q) * L.ld + h * hd + ch, oacc[v] / qsum[ql]);
        }
    __syncthreads ();                                    // qsum is reused by the next tile of this workgroup
}

// ---------------------------------------------------------------------------------------------
// Dispatch: the device-side counterpart of the switch in the reference's dse_schedule
// (reference src/dse.c:39-79).  `t` = tile index inside the layer, row-tile fastest
// (reference src/apu_nasm.c:1218-1224).
// ---------------------------------------------------------------------------------------------
// A wave-uniform copy of a layer descriptor in scalar registers.  Every value derived from the descriptor must
// be known to be uniform: otherwise buffer descriptors get rebuilt in a per-lane "waterfall" loop around each
// access and all tile-level control flow runs on the vector unit.
//
// scalar_layer reads a descriptor in device memory through the scalar data cache (read-only use: descriptors
// are written by the host before the launch and never by a kernel), 64 dwords in a handful of wide scalar
// loads straight into scalar registers.  `g` must be the same for all lanes.
__device__ __forceinline__ aspen_hip_layer_t scalar_layer (const aspen_hip_layer_t *g)
{
    constexpr int W = sizeof (aspen_hip_layer_t) / 4;
    static_assert (sizeof (aspen_hip_layer_t) % 4 == 0, "descriptor is a whole number of dwords");
    const uint64_t p = (uint64_t)g;
    // (the builtin returns int: without the casts the low half would be sign-extended over the high one)
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane ((uint32_t)p), hi = (uint32_t)__builtin_amdgcn_readfirstlane ((uint32_t)(p >> 32));
    uint64_t up = ((uint64_t)hi << 32) | (uint64_t)lo;
    // Every call loads afresh: the compiler may not merge the loads of two calls (and so keep all 64 dwords in
    // registers from the first use of a descriptor to the last), because it cannot see that `up` is unchanged.
    asm volatile ("" : "+s" (up));
    const uint32_t __attribute__ ((address_space (4))) *src = (const uint32_t __attribute__ ((address_space (4))) *)up;
    uint32_t w[W];
    #pragma unroll
    for (int i = 0; i < W; i++) w[i] = src[i];
    aspen_hip_layer_t L;
    __builtin_memcpy (&L, w, sizeof (aspen_hip_layer_t));
    return L;
}
// uniform_layer does the same for a descriptor the compiler already holds (a kernel argument).
__device__ __forceinline__ aspen_hip_layer_t uniform_layer (const aspen_hip_layer_t &Lg)
{
    constexpr int W = sizeof (aspen_hip_layer_t) / 4;
    uint32_t w[W];
    __builtin_memcpy (w, &Lg, sizeof (aspen_hip_layer_t));
    #pragma unroll
    for (int i = 0; i < W; i++) w[i] = __builtin_amdgcn_readfirstlane (w[i]);
    aspen_hip_layer_t L;
    __builtin_memcpy (&L, w, sizeof (aspen_hip_layer_t));
    return L;
}

// Counts this workgroup's arrival in its split-K group; true for the last of the `splits` members.  The
// group's (write-through) stores must have been acknowledged before an arrival is counted: the last
// one reads them.  The counter only ever grows by `splits` per run, so it needs no reset between runs.
__device__ __forceinline__ bool splitk_arrived_last (uint32_t *counter, uint32_t splits, float *smem)
{
    asm volatile ("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads ();
    uint32_t *flag = reinterpret_cast<uint32_t *> (smem);
    if (tile_thread () == 0)
        *flag = __hip_atomic_fetch_add (counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads ();
    const uint32_t before = __builtin_amdgcn_readfirstlane (*flag);
    __syncthreads ();                       // the flag's word is LDS the next tile reuses
    return before % splits == splits - 1;
}

// ---------------------------------------------------------------------------------------------
// The narrow contraction tile: 32 channels x 32 columns, the four wavefronts of the workgroup splitting the K axis
// between them.  For graphs that are bound by the latency of their dependency chains (one image through a deep
// network): a layer of a few dozen 64 x 64 tiles with long K loops becomes a few hundred short ones, so that a
// dependency level keeps every compute unit busy for one or two microseconds instead of a quarter of them for
// eight.  Throughput per workgroup does not matter here, so there is nothing to share between wavefronts and
// nothing is staged through LDS: a lane reads its operands from memory in the layout the matrix instruction wants
// (row = lane % 32, four consecutive K values at (lane / 32) * 4 of every 8: v_mfma_f32_32x32x2_f32 pairs the two
// half-waves' values, and both operands use the same pairing, so the K order inside a slice is immaterial), the
// K loop has no barrier, and the four partial sums meet in LDS once.  A layer can additionally be cut along K across
// workgroups (`slice` >= 0) exactly like the 64 x 64 shape, with blocks of 32 x 32 sums in the threads' own order.
// Operands: weights [.][Kp]; activations read in place (DIRECT) or gathered by stepping through the taps (a
// convolution or FC layer over channels that are a multiple of the slice width).
// ---------------------------------------------------------------------------------------------
#define VAR3_BM 32
#define VAR3_BN 32
#define NARROW_TILE_FLOATS (VAR3_BM * VAR3_BN)
#define NARROW_ROW 36          // floats per staged row of a wavefront's partial sums

// what a thread of a narrow tile owns after the four wavefronts' sums have met: channels c .. c+3 of column n
struct narrow_piece_t { uint32_t n, c; };
__device__ __forceinline__ narrow_piece_t narrow_piece (uint32_t tid) { return {tid >> 3, (tid & 7u) * 4u}; }

// bias, activation, store and fused shortcut of one thread's piece; `sc` = the shortcut operand's piece when `have_sc`
template <int COH>
__device__ __forceinline__ void narrow_finish_piece (const aspen_hip_layer_t &L, uint32_t tn, uint32_t tm, uint32_t tid, float4 v, float4 bias, bool have_bias,
    float4 sc, bool have_sc)
{
    const narrow_piece_t pc = narrow_piece (tid);
    const uint32_t n = tn * VAR3_BN + pc.n, m = tm * VAR3_BM + pc.c;
    if (n >= L.N || m >= L.M) return;
    const uint32_t left = L.M - m;
    ActView<COH> out;
    out.init (L.out, L.N, L.ld);
    if (!have_bias && L.bias)
    {
        bias.x = gld1 (L.bias + m);
        if (left > 1) bias.y = gld1 (L.bias + m + 1);
        if (left > 2) bias.z = gld1 (L.bias + m + 2);
        if (left > 3) bias.w = gld1 (L.bias + m + 3);
    }
    v.x += bias.x; v.y += bias.y; v.z += bias.z; v.w += bias.w;
    v = act4 (v, L.act);
    const bool fuse = L.fuse_out != nullptr, keep = !(fuse && L.fuse_discard);
    const uint32_t o = n * L.ld + m;
    if (left >= 4)
    {
        if (keep) out.st4 (o, v);
        if (fuse)
        {
            ActView<COH> fout;
            fout.init (L.fuse_out, L.N, L.ld);
            if (!have_sc) { ActView<COH> fin; fin.init (L.fuse_in, L.N, L.fuse_ld_in); sc = fin.ld4 (n * L.fuse_ld_in + m); }
            v.x += sc.x; v.y += sc.y; v.z += sc.z; v.w += sc.w;
            fout.st4 (o, act4 (v, L.fuse_act));
        }
    }
    else
    {
        if (keep) { out.st1 (o, v.x); if (left > 1) out.st1 (o + 1, v.y); if (left > 2) out.st1 (o + 2, v.z); }
        if (fuse)
        {
            ActView<COH> fin, fout;
            fin.init (L.fuse_in, L.N, L.fuse_ld_in); fout.init (L.fuse_out, L.N, L.ld);
            fused_shortcut<COH> (L, fin, fout, v, n, m, left);
        }
    }
}

// sum of the slices' blocks of output tile t (in slice order, whoever runs it), then the tile's epilogue
template <int COH>
__device__ __forceinline__ void narrow_gather_finish (const aspen_hip_layer_t &L, uint32_t t, uint32_t tn, uint32_t tm)
{
    const uint32_t tid = tile_thread ();
    const uint32_t tiles = L.tiles_m * L.tiles_n, sstride = tiles * NARROW_TILE_FLOATS, last = L.splits - 1;
    ActView<COH> part;
    part.init (L.partial, L.splits * tiles, NARROW_TILE_FLOATS);
    const uint32_t base = t * NARROW_TILE_FLOATS + tid * 4;
    float4 v = make_float4 (0.f, 0.f, 0.f, 0.f);
    constexpr uint32_t BATCH = 8;       // requests in flight per thread: the blocks come from other compute units' tiles
    for (uint32_t s0 = 0; s0 < L.splits; s0 += BATCH)
    {
        float4 p[BATCH];
        #pragma unroll
        for (uint32_t j = 0; j < BATCH; j++) p[j] = part.ld4 (base + min (s0 + j, last) * sstride);
        #pragma unroll
        for (uint32_t j = 0; j < BATCH; j++)
        {
            const bool use = s0 + j <= last;
            v.x += use ? p[j].x : 0.f; v.y += use ? p[j].y : 0.f; v.z += use ? p[j].z : 0.f; v.w += use ? p[j].w : 0.f;
        }
    }
    narrow_finish_piece<COH> (L, tn, tm, tid, v, make_float4 (0.f, 0.f, 0.f, 0.f), false, make_float4 (0.f, 0.f, 0.f, 0.f), false);
}

// Returns the thread's piece of the tile's sums over the K slices [kbase, kbase + kiters).
// PF > 0 (kernels that start a tile before its parents have finished, with PF * 16 KB of LDS per workgroup): the
// weights of a wavefront's first PF slices are requested BEFORE `ready ()`, straight from memory into LDS
// (buffer_load ... lds: lane l's 16 bytes land at block + 16 l, so a lane later reads back exactly the fragment it
// asked for; LDS serves as a per-lane buffer that costs no registers), and the activations of the first NARROW_B_WINDOW
// of them are all requested together right after it, the rest as the window's registers come free: a tile of up to PF
// slices per wavefront pays for one trip to memory after its parents have finished.  Slices beyond PF (and all slices when PF = 0) go through registers, two in flight.
#define NARROW_PF_SLICES 4
#define NARROW_B_WINDOW 4           // slices of activations in flight in registers
#define NARROW_PF_SMEM_BYTES (4 * NARROW_PF_SLICES * 4 * 1024)
template <int COH, int PF, class Descriptor, class Ready>
__device__ __forceinline__ float4 narrow_mainloop (const aspen_hip_layer_t &L, Descriptor descriptor, uint32_t tn, uint32_t tm, int kbase, int kiters,
    float *smem, Ready ready)
{
    const uint32_t tid = tile_thread (), lane = tid & 63, wave = __builtin_amdgcn_readfirstlane (tid >> 6);
    const uint32_t row = lane & 31, khalf = (lane >> 5) * 4;
    // this wavefront's share of the slices: a contiguous quarter
    const int per = (kiters + 3) >> 2, w0 = min ((int)wave * per, kiters), cnt = min (per, kiters - w0), first = kbase + w0;
    // weights: one uniform base, 32-bit byte offsets
    const float *wptr = descriptor ().weight;
    const char __attribute__ ((address_space (1))) *wbase = (const char __attribute__ ((address_space (1))) *)wptr;
    const uint32_t aoff = (((tm * VAR3_BM + row) * L.Kp) + (uint32_t)first * GEMM_BK + khalf) * 4u;
    ActView<COH> in;
    in.init (descriptor ().in0, L.in0_columns, L.ld0);
    const bool direct = L.direct == ASPEN_HIP_OPERAND_DIRECT;
    uint32_t n = tn * VAR3_BN + row;
    n = n < L.N ? n : L.N - 1;
    // activation operand: DIRECT = the parent's column; else the top-left input pixel of output position n and the
    // tap / channel the first slice starts at (stepped from there, as ConvLoader does)
    int32_t bbase, ih0 = 0, iw0 = 0;
    uint32_t kh = 0, kw = 0, c = 0;
    if (direct) bbase = (int32_t)(n * L.ld0 + (uint32_t)first * GEMM_BK + khalf);
    else
    {
        const uint32_t ohw = L.OH * L.OW;
        const uint32_t b = fast_div (n, L.div_ohw), rem = n - b * ohw, oh = fast_div (rem, L.div_ow), ow = rem - oh * L.OW;
        ih0 = (int32_t)(oh * L.stride) - (int32_t)L.pad;
        iw0 = (int32_t)(ow * L.stride) - (int32_t)L.pad;
        bbase = ((int32_t)(b * L.IH) + ih0) * (int32_t)L.IW * (int32_t)L.ld0 + iw0 * (int32_t)L.ld0 + (int32_t)khalf;
        // (K order: channel block, kh, kw, channel in block; see ConvLoader)
        const uint32_t taps = L.KH * L.KW, block = (uint32_t)first / taps, tap = (uint32_t)first - block * taps;
        c = block * GEMM_BK;
        kh = tap / L.KW; kw = tap - kh * L.KW;
    }
    const uint32_t IH = L.IH, IW = L.IW, KH = L.KH, KW = L.KW, ld0 = L.ld0;
    auto load_a = [&] (int i, float4 (&a)[4])
    {
        #pragma unroll
        for (int sub = 0; sub < 4; sub++)
        {
            const floatx4 x = *(const floatx4 __attribute__ ((address_space (1))) *)(wbase + (aoff + (uint32_t)i * (GEMM_BK * 4u) + (uint32_t)sub * 32u));
            a[sub] = make_float4 (x[0], x[1], x[2], x[3]);
        }
    };
    // slices are asked for in ascending order: the tap position is stepped
    auto load_b = [&] (int i, float4 (&bv)[4])
    {
        if (direct)
        {
            #pragma unroll
            for (int sub = 0; sub < 4; sub++) bv[sub] = in.ld4 ((uint32_t)(bbase + i * GEMM_BK + sub * 8));
        }
        else
        {
            const int32_t off = (int32_t)((kh * IW + kw) * ld0 + c);
            const bool ok = (uint32_t)(ih0 + (int32_t)kh) < IH && (uint32_t)(iw0 + (int32_t)kw) < IW;
            #pragma unroll
            for (int sub = 0; sub < 4; sub++) bv[sub] = in.ld4_if ((uint32_t)(bbase + off + sub * 8), ok);
            if (++kw == KW) { kw = 0; if (++kh == KH) { kh = 0; c += GEMM_BK; } }
        }
    };
    floatx16 acc;
    #pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = 0.f;
    auto mfmas = [&] (const float4 (&a)[4], const float4 (&bv)[4])
    {
        #pragma unroll
        for (int sub = 0; sub < 4; sub++)
        {
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32 (bv[sub].x, a[sub].x, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32 (bv[sub].y, a[sub].y, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32 (bv[sub].z, a[sub].z, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32 (bv[sub].w, a[sub].w, acc, 0, 0, 0);
        }
    };
    constexpr uint32_t REGION = PF > 0 ? PF * 1024u : (uint32_t)(VAR3_BN * NARROW_ROW);     // floats of LDS per wavefront
    float *mine = smem + wave * REGION;
    int done = 0;       // slices of this wavefront's share that are finished
    float4 a0[4], a1[4], b0[4], b1[4];
    if constexpr (PF > 0)
    {
        const uint32_t Mp = (L.M + 127u) / 128u * 128u;
        const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc ((void *)wptr, 0, (int)(Mp * L.Kp * 4u), 0x00020000);
        #pragma unroll
        for (int i = 0; i < PF; i++)
            if (i < cnt)
            {
                #pragma unroll
                for (int sub = 0; sub < 4; sub++)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds (wr, (__attribute__ ((address_space (3))) void *)(mine + (i * 4 + sub) * 256), 16,
                        (int)(aoff + (uint32_t)i * (GEMM_BK * 4u) + (uint32_t)sub * 32u), 0, 0, 0);
            }
        ready ();
        // one straight-line body per number of prefetched slices (wave-uniform): every activation request is issued
        // before the first fragment is read back, so the slices' trips to memory overlap
        auto body = [&] (auto count)
        {
            constexpr int C = decltype (count)::value, W = C < NARROW_B_WINDOW ? C : NARROW_B_WINDOW;
            float4 bq[W][4];
            #pragma unroll
            for (int i = 0; i < W; i++) load_b (i, bq[i]);
            #pragma unroll
            for (int i = 0; i < C; i++)
            {
                float4 af[4];
                #pragma unroll
                for (int sub = 0; sub < 4; sub++) af[sub] = ld4 (mine + (i * 4 + sub) * 256 + lane * 4);
                mfmas (af, bq[i % W]);
                if (i + W < C) load_b (i + W, bq[i % W]);       // the window moves on: this slice's registers take the slice W ahead
            }
        };
        static_assert (PF == 4, "one case per prefetched slice count");
        const int pre = __builtin_amdgcn_readfirstlane (min (cnt, PF));
        if (pre == 4) body (std::integral_constant<int, 4> ());
        else if (pre == 3) body (std::integral_constant<int, 3> ());
        else if (pre == 2) body (std::integral_constant<int, 2> ());
        else if (pre == 1) body (std::integral_constant<int, 1> ());
        done = min (cnt, PF);
        if (done < cnt) { load_a (done, a0); load_b (done, b0); }
        if (done + 1 < cnt) { load_a (done + 1, a1); load_b (done + 1, b1); }
    }
    else
    {
        // two slices in flight: set 0 holds the even, set 1 the odd ones of this wavefront's share
        if (cnt > 0) load_a (0, a0);
        if (cnt > 1) load_a (1, a1);
        ready ();
        if (cnt > 0) load_b (0, b0);
        if (cnt > 1) load_b (1, b1);
    }
    for (int i = done; i < cnt; i += 2)
    {
        mfmas (a0, b0);
        if (i + 2 < cnt) { load_a (i + 2, a0); load_b (i + 2, b0); }
        if (i + 1 < cnt)
        {
            mfmas (a1, b1);
            if (i + 3 < cnt) { load_a (i + 3, a1); load_b (i + 3, b1); }
        }
    }
    // the four wavefronts' sums meet in LDS: [wave][column][NARROW_ROW] (a wavefront's own region, which it has read empty)
    #pragma unroll
    for (int v = 0; v < 16; v++) mine[ACC_N (0, 0, v, lane) * NARROW_ROW + row] = acc[v];
    __syncthreads ();
    const narrow_piece_t pc = narrow_piece (tid);
    float4 sum = ld4 (smem + pc.n * NARROW_ROW + pc.c);
    #pragma unroll
    for (int w = 1; w < 4; w++)
    {
        const float4 x = ld4 (smem + w * REGION + pc.n * NARROW_ROW + pc.c);
        sum.x += x.x; sum.y += x.y; sum.z += x.z; sum.w += x.w;
    }
    return sum;
}

// One narrow tile; returns false for a split-K member that was not the last of its group.
template <int COH, int PF, class Descriptor, class Arrivals, class Ready>
__device__ __forceinline__ bool narrow_tile (const aspen_hip_layer_t &L, Descriptor descriptor, uint32_t t, uint32_t tn, uint32_t tm, int slice, uint32_t group,
    float *smem, Arrivals arrivals, Ready ready)
{
    const uint32_t tid = tile_thread ();
    int kbase = 0, kiters = (int)(L.Kp / GEMM_BK);
    if (slice >= 0)
    {
        kbase = slice * (int)L.kiters_per_split;
        kiters = min ((int)L.kiters_per_split, kiters - kbase);
    }
    // the bias is a weight: requested before the wait for the parents
    const narrow_piece_t pc = narrow_piece (tid);
    const uint32_t m = tm * VAR3_BM + pc.c, n = tn * VAR3_BN + pc.n;
    const bool whole = slice < 0 && m + 4 <= L.M && n < L.N;
    float4 bias = make_float4 (0.f, 0.f, 0.f, 0.f), sc = bias;
    if (whole && L.bias) bias = gld4 (L.bias + m);
    bool have_sc = false;
    const auto ready_then_shortcut = [&] ()
    {
        ready ();
        // an unsplit tile's shortcut operand is an activation its dependency counter covers: requested with the first slice
        if (whole && L.fuse_out != nullptr)
        {
            ActView<COH> fin;
            fin.init (L.fuse_in, L.N, L.fuse_ld_in);
            sc = fin.ld4 (n * L.fuse_ld_in + m);
            have_sc = true;
        }
    };
    const float4 sum = narrow_mainloop<COH, PF> (L, descriptor, tn, tm, kbase, kiters, smem, ready_then_shortcut);
    if (COH) tile_phase_lap (9);
    if (slice < 0)
    {
        narrow_finish_piece<COH> (L, tn, tm, tid, sum, bias, whole, sc, have_sc);
        if (COH) tile_phase_lap (10);
        return true;
    }
    {
        const uint32_t tiles = L.tiles_m * L.tiles_n;
        ActView<COH> part;
        part.init (L.partial, L.splits * tiles, NARROW_TILE_FLOATS);
        part.st4 (((uint32_t)slice * tiles + t) * NARROW_TILE_FLOATS + tid * 4, sum);
    }
    if (COH) tile_phase_lap (10);
    uint32_t *counters = arrivals ();
    if (counters == nullptr || !splitk_arrived_last (counters + group, L.splits, smem)) { if (COH) tile_phase_lap (11); return false; }
    narrow_gather_finish<COH> (L, t, tn, tm);
    if (COH) tile_phase_lap (11);
    return true;
}

// Split-K reduction of output tile t of the layer as a tile of its own (launch-per-layer mode).
template <int COH>
__device__ __forceinline__ void finish_tile (const aspen_hip_layer_t &L, uint32_t t, float *smem)
{
    t = __builtin_amdgcn_readfirstlane (t);
    const uint32_t tn = fast_div (t, L.div_tiles_m);
    if (L.variant == ASPEN_HIP_GEMM_NARROW) { narrow_gather_finish<COH> (L, t, tn, t - tn * L.tiles_m); return; }
    shortcut_prefetch_t pre;
    pre.have = pre.have_shortcut = false;
    const bool tall = L.variant == ASPEN_HIP_GEMM_TALL;
    splitk_gather<COH> (L, t, smem, tall);
    contraction_epilogue<COH, true> (L, tn, t - tn * L.tiles_m, smem, tall ? 5 : 4, tall ? VAR4_BN : VAR2_BN, pre);
}

// Runs tile t of the layer.  `descriptor ()` yields a wave-uniform copy of the layer's descriptor (scalar_layer /
// uniform_layer); a contraction tile asks for it a second time behind its K loop, so that what only the
// epilogue needs does not occupy scalar registers while the loop runs.  `arrivals ()` yields the graph's array of zero-initialised counters, one per
// tile (used at the index of a split-K group's first tile); it is a callable so that the pointer is
// fetched where it is needed instead of occupying registers while the tile runs.  Returns false for
// a split-K partial tile that was not the last of its group to finish: the output tile is not
// complete yet and nothing may be released.
// `ready ()` returns once the tile's parents have finished; it is called after whatever set-up does not touch an
// activation (contraction tiles: descriptor, index arithmetic, first weight requests), right before the first
// activation is requested.  Kernels that only start tiles whose parents have finished pass nothing.
// Row groups: under the large shape a layer with a short K axis may give a workgroup SEVERAL row tiles of one column
// block (tile_m = 2 or 4 times the shape's 128 rows): such tiles are all set-up, first fetch and epilogue, and a
// workgroup that works through its column block's row tiles pays one scheduling step for all of them and finds the
// activation block in its caches from the second one on.  The caller runs the tile once per row tile, row_rep = 0, 1, ...
// while *more_rows comes back true (the tile code itself stays one straight pass: a loop around it here made the
// compiler duplicate and spill the persistent kernel's K loops).
template <int COH, unsigned FEAT = TILES_ALL, int NARROW_PF = 0, class Descriptor, class Arrivals, class Ready = NoHook>
__device__ __forceinline__ bool run_tile (Descriptor descriptor, uint32_t t, bool t_counts_from_graph_start, float *smem, Arrivals arrivals, Ready ready = Ready (),
    uint32_t row_rep = 0, bool *more_rows = nullptr)
{
    const aspen_hip_layer_t L = descriptor ();
    t = __builtin_amdgcn_readfirstlane (t);
    if (t_counts_from_graph_start) t -= L.ninst_start;
    int slice = -1;
    uint32_t group = 0;
    if (L.splits > 1)
    {
        const uint32_t q = fast_div (t, L.div_splits);
        slice = (int)(t - q * L.splits);
        group = L.ninst_start + t - (uint32_t)slice;
        t = q;
    }
    const uint32_t tn = fast_div (t, L.div_tiles_m);
    uint32_t tm = t - tn * L.tiles_m;
    switch (L.type)
    {
    case CONV_LAYER: case FC_LAYER: case MATMUL_LAYER:
    {
        uint32_t c4_log2, bn;
        shortcut_prefetch_t pre;
        pre.have = pre.have_shortcut = false;
        c4_log2 = 4; bn = VAR2_BN;
        if constexpr ((FEAT & TILES_NARROW) != 0)
        {
            if (L.variant == ASPEN_HIP_GEMM_NARROW) return narrow_tile<COH, NARROW_PF> (L, descriptor, t, tn, tm, slice, group, smem, arrivals, ready);
        }
        if ((FEAT & TILES_LARGE) && L.variant == ASPEN_HIP_GEMM_LARGE)
        {
            const uint32_t reps = L.tile_m / VAR0_BM;
            if (reps > 1)
            {
                if (row_rep) __syncthreads ();      // the previous row tile's epilogue has read the stage this one refills
                tm = tm * reps + row_rep;
                if (more_rows) *more_rows = row_rep + 1 < reps;
            }
            const auto ready_first = [&] () { if (row_rep == 0) ready (); };
            contraction_mainloop<VAR0_BM, VAR0_BN, 2, 2, VAR0_DEPTH, COH, FEAT> (L, descriptor, tn, tm, -1, smem, pre, ready_first);
            c4_log2 = 5; bn = VAR0_BN;
        }
        else if ((FEAT & TILES_WIDE) && L.variant == ASPEN_HIP_GEMM_WIDE) { contraction_mainloop<VAR1_BM, VAR1_BN, 2, 2, VAR1_DEPTH, COH, FEAT> (L, descriptor, tn, tm, -1, smem, pre, ready); bn = VAR1_BN; }
        else if ((FEAT & TILES_TALL) && L.variant == ASPEN_HIP_GEMM_TALL) { contraction_mainloop<VAR4_BM, VAR4_BN, 4, 1, VAR4_DEPTH, COH, FEAT> (L, descriptor, tn, tm, slice, smem, pre, ready); c4_log2 = 5; bn = VAR4_BN; }
        else if (FEAT & TILES_SMALL)
        {
            // two K slices in flight for the matmul layers of transformers, one for convolutional networks (see VAR2_DEPTH)
            bool deep = false;
            if constexpr ((FEAT & TILES_NORM) != 0) deep = (FEAT & TILES_GATHER) == 0 || L.type == MATMUL_LAYER;
            if constexpr ((FEAT & TILES_NORM) != 0) { if (deep) contraction_mainloop<VAR2_BM, VAR2_BN, 2, 2, VAR2_DEPTH, COH, FEAT> (L, descriptor, tn, tm, slice, smem, pre, ready); }
            if constexpr ((FEAT & TILES_GATHER) != 0) { if (!deep) contraction_mainloop<VAR2_BM, VAR2_BN, 2, 2, 1, COH, FEAT> (L, descriptor, tn, tm, slice, smem, pre, ready); }
        }
        
        const aspen_hip_layer_t E = descriptor ();
        if (slice >= 0)
        {
            // split-K: every slice has written its sums; whoever arrives last adds them up and finishes the tile.
            // Without counters (one launch per layer: stores of a launch are not visible across XCDs before it
            // ends) that is left to a second launch, see finish_tile.
            if (COH) tile_phase_lap (10);
            uint32_t *counters = arrivals ();
            if (counters == nullptr || !splitk_arrived_last (counters + group, E.splits, smem)) { if (COH) tile_phase_lap (11); return false; }
            splitk_gather<COH> (E, t, smem, c4_log2 == 5);       // (of the shapes cut along K only the tall one has 128 channels)
        }
        contraction_epilogue<COH, (FEAT & TILES_NORM) != 0> (E, tn, tm, smem, c4_log2, bn, pre);
        if (COH) tile_phase_lap (slice >= 0 ? 11 : 10);
        break;
    }
    case RESIDUAL_LAYER:    if constexpr ((FEAT & TILES_RESIDUAL) != 0) { ready (); tile_residual<COH> (L, tn); } break;
    case MAXPOOL_LAYER:     if constexpr ((FEAT & TILES_POOL) != 0) { ready (); tile_pool<true, COH> (L, tn, tm); } break;
    case AVGPOOL_LAYER:     if constexpr ((FEAT & TILES_POOL) != 0) { ready (); tile_pool<false, COH> (L, tn, tm); } break;
    case YOLO_LAYER:        if constexpr ((FEAT & TILES_YOLO) != 0) { ready (); tile_yolo<COH> (L, tn); } break;
    case APPEND_LAYER:      if constexpr ((FEAT & TILES_YOLO) != 0) { ready (); tile_append<COH> (L, tn); } break;
    case LAYERNORM_LAYER:   if constexpr ((FEAT & TILES_NORM) != 0) { ready (); tile_layernorm<COH> (L, tn); } break;
    case SOFTMAX_LAYER:     if constexpr ((FEAT & TILES_NORM) != 0) { ready (); tile_softmax<COH> (L, tn); } break;
    case K_ATTENTION_LAYER: if constexpr ((FEAT & TILES_ATTENTION) != 0) { ready (); tile_k_attention<COH> (L, tn, smem); } break;
    case V_ATTENTION_LAYER:
        if constexpr ((FEAT & TILES_ATTENTION) != 0)
        {
            ready ();
            if (L.direct == ASPEN_HIP_ATTENTION_FUSED) tile_fused_attention<COH> (L, tn, tm, smem);
            else tile_v_attention<COH> (L, tn, tm, smem);
        }
        break;
    default: break;
    }
    return true;
}
