/*
 * aspen_oracle.c -- TEST INFRASTRUCTURE ONLY (the parity oracle).
 *
 * A from-scratch CPU restatement of the reference's tile arithmetic, written
 * per whole layer on dense matrices.  The product library never links, loads
 * or calls this file; only tests/, __graft_entry__.smoke() and bench.py's
 * cpu_baseline leg do, and only as the checker / the timed baseline.
 *
 * Activations are "out_mat" matrices as in the reference: W columns of ld
 * floats, rows = channels (NHWC with a padded channel run, reference
 * src/apu_nasm.c:950-1017, :1226-1262).  Every function takes explicit leading
 * dimensions so the caller may use dense (ld == H) or padded storage.
 *
 * Pinning (what each function was checked against; see tests/test_oracle_*.py):
 *   pack_weight / sgemm_packed : brute-force triple loop incl. M%8, odd N, odd K;
 *                                reference's packed tensors via oracle/_ref
 *   conv2d / maxpool / avgpool / fc / matmul / layernorm / residual / softmax /
 *   k_attention / v_attention  : torch.nn.functional on CPU (library routine) and
 *                                the compiled reference (oracle/_ref) per layer
 *   activate                   : closed forms + torch gelu (erf and tanh variants)
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <stdint.h>

typedef float v8f __attribute__ ((vector_size (32), aligned (4)));

/* LAYER_ACT numbering of the reference (include/aspen.h:63). */
enum { ACT_NONE = 0, ACT_SIGMOID, ACT_LINEAR, ACT_TANH, ACT_RELU, ACT_LEAKY, ACT_ELU, ACT_SELU, ACT_GELU, ACT_GELU_ACC };

/* reference src/naive_kernels.c:11-57 (same expressions, same double promotions) */
void oracle_activate (float *x, unsigned int n, int act)
{
    unsigned int i;
    switch (act)
    {
    case ACT_NONE: case ACT_LINEAR: return;
    case ACT_RELU:   for (i = 0; i < n; i++) x[i] = x[i] > 0 ? x[i] : 0; return;
    case ACT_LEAKY:  for (i = 0; i < n; i++) x[i] = x[i] > 0 ? x[i] : 0.1 * x[i]; return;
    case ACT_ELU:    for (i = 0; i < n; i++) x[i] = x[i] > 0 ? x[i] : 0.1 * (exp (x[i]) - 1); return;
    case ACT_SELU:   for (i = 0; i < n; i++) x[i] = x[i] > 0 ? 1.0507 * x[i] : 1.0507 * 1.67326 * (exp (x[i]) - 1); return;
    case ACT_SIGMOID:for (i = 0; i < n; i++) x[i] = 1 / (1 + exp (-x[i])); return;
    case ACT_TANH:   for (i = 0; i < n; i++) x[i] = tanh (x[i]); return;
    case ACT_GELU:   for (i = 0; i < n; i++) x[i] = 0.5 * x[i] * (1 + erff (x[i] * 0.7071067811865475f)); return;
    case ACT_GELU_ACC:
        for (i = 0; i < n; i++)
            x[i] = 0.5 * x[i] * (1 + tanhf (0.7978845608028654f * (x[i] + 0.044715 * x[i] * x[i] * x[i])));
        return;
    default: return;
    }
}

/* Weight packing [M][K] row-major -> [ceil(M/8)][K][8]; element (m,k) lands at
   ((m/8)*K + k)*8 + m%8 (reference src/apu.c:14-40, restated at src/naive_kernels.c:575).
   Rows beyond M are zero.  `packed` must hold ceil(M/8)*K*8 floats. */
void oracle_pack_weight (const float *w, float *packed, unsigned int M, unsigned int K)
{
    unsigned int Mp = (M + 7) / 8;
    memset (packed, 0, (size_t)Mp * K * 8 * sizeof (float));
    for (unsigned int m = 0; m < M; m++)
        for (unsigned int k = 0; k < K; k++)
            packed[((size_t)(m / 8) * K + k) * 8 + (m % 8)] = w[(size_t)m * K + k];
}

/* PyTorch conv weight [OC][IC][KH][KW] -> [OC][(kh*KW+kw)*IC + ic] (reference src/apu.c:16). */
void oracle_conv_weight_to_hwc (const float *oihw, float *ohwi, unsigned int OC, unsigned int IC, unsigned int KH, unsigned int KW)
{
    for (unsigned int o = 0; o < OC; o++)
        for (unsigned int i = 0; i < IC; i++)
            for (unsigned int h = 0; h < KH; h++)
                for (unsigned int w = 0; w < KW; w++)
                    ohwi[((size_t)o * KH * KW + h * KW + w) * IC + i] = oihw[(((size_t)o * IC + i) * KH + h) * KW + w];
}

/* C[n*ldc + m] += sum_k A[((m/8)*lda + k)*8 + m%8] * B[n*ldb + k], k ascending
   (reference src/avx2_kernels.c:526-1045; 8-row vector = one packed A group). */
void oracle_sgemm_packed (unsigned int M, unsigned int N, unsigned int K,
    const float *A, unsigned int lda, const float *B, unsigned int ldb, float *C, unsigned int ldc)
{
    unsigned int m8;
    for (m8 = 0; m8 * 8 < M; m8++)
    {
        const float *Ap = A + (size_t)m8 * lda * 8;
        unsigned int rows = (M - m8 * 8) < 8 ? (M - m8 * 8) : 8;
        unsigned int n = 0;
        for (; n + 4 <= N; n += 4)
        {
            v8f c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
            const float *b0 = B + (size_t)n * ldb, *b1 = b0 + ldb, *b2 = b1 + ldb, *b3 = b2 + ldb;
            for (unsigned int k = 0; k < K; k++)
            {
                v8f a = *(const v8f *)(Ap + (size_t)k * 8);
                c0 += a * b0[k]; c1 += a * b1[k]; c2 += a * b2[k]; c3 += a * b3[k];
            }
            for (unsigned int j = 0; j < rows; j++)
            {
                C[(size_t)(n + 0) * ldc + m8 * 8 + j] += c0[j];
                C[(size_t)(n + 1) * ldc + m8 * 8 + j] += c1[j];
                C[(size_t)(n + 2) * ldc + m8 * 8 + j] += c2[j];
                C[(size_t)(n + 3) * ldc + m8 * 8 + j] += c3[j];
            }
        }
        for (; n < N; n++)
        {
            v8f c0 = {0};
            const float *b0 = B + (size_t)n * ldb;
            for (unsigned int k = 0; k < K; k++)
                c0 += *(const v8f *)(Ap + (size_t)k * 8) * b0[k];
            for (unsigned int j = 0; j < rows; j++)
                C[(size_t)n * ldc + m8 * 8 + j] += c0[j];
        }
    }
}

static void bias_act (float *C, unsigned int ldc, unsigned int M, unsigned int N, const float *bias, int act)
{
    for (unsigned int n = 0; n < N; n++)
    {
        float *v = C + (size_t)n * ldc;
        if (bias != NULL)
            for (unsigned int m = 0; m < M; m++)
                v[m] += bias[m];
        oracle_activate (v, M, act);
    }
}

#define COLS_PER_BLOCK 48

/* conv as im2col + packed GEMM, epilogue order zero -> accumulate -> +bias -> activation
   (reference src/tiled_kernels.c:161-297; gather = prepare_input :3-45 + load_im2col_ptr :104-159).
   in : [B*IH*IW] columns of ldin floats (IC used); out: [B*OH*OW] columns of ldout floats (OC used).
   Wp : packed [ceil(OC/8)][K][8], K = KH*KW*IC ordered (kh, kw, ic). */
void oracle_conv2d (const float *in, unsigned int ldin, const float *Wp, const float *bias,
    float *out, unsigned int ldout, unsigned int B, unsigned int IH, unsigned int IW, unsigned int IC,
    unsigned int OC, unsigned int KH, unsigned int KW, unsigned int stride, unsigned int pad, int act)
{
    const unsigned int OH = (IH + 2 * pad - (KH - 1) - 1) / stride + 1;
    const unsigned int OW = (IW + 2 * pad - (KW - 1) - 1) / stride + 1;
    const unsigned int K = KH * KW * IC;
    const long N = (long)B * OH * OW;
    #pragma omp parallel
    {
        float *panel = malloc ((size_t)COLS_PER_BLOCK * K * sizeof (float));
        #pragma omp for schedule(dynamic, 4)
        for (long n0 = 0; n0 < N; n0 += COLS_PER_BLOCK)
        {
            unsigned int nb = (N - n0) < COLS_PER_BLOCK ? (unsigned int)(N - n0) : COLS_PER_BLOCK;
            for (unsigned int nn = 0; nn < nb; nn++)
            {
                long col = n0 + nn;
                unsigned int b = col / (OH * OW), oh = (col % (OH * OW)) / OW, ow = col % OW;
                float *row = panel + (size_t)nn * K;
                for (unsigned int kh = 0; kh < KH; kh++)
                    for (unsigned int kw = 0; kw < KW; kw++)
                    {
                        int ih = (int)(oh * stride + kh) - (int)pad, iw = (int)(ow * stride + kw) - (int)pad;
                        float *dst = row + (size_t)(kh * KW + kw) * IC;
                        if (ih < 0 || ih >= (int)IH || iw < 0 || iw >= (int)IW)
                            memset (dst, 0, IC * sizeof (float));
                        else
                            memcpy (dst, in + ((size_t)b * IH * IW + (size_t)ih * IW + iw) * ldin, IC * sizeof (float));
                    }
                memset (out + (size_t)col * ldout, 0, OC * sizeof (float));
            }
            oracle_sgemm_packed (OC, nb, K, Wp, K, panel, K, out + (size_t)n0 * ldout, ldout);
            bias_act (out + (size_t)n0 * ldout, ldout, OC, nb, bias, act);
        }
        free (panel);
    }
}

/* matmul: B operand read in place from the parent (reference src/tiled_kernels.c:299-409). */
void oracle_matmul (const float *in, unsigned int ldin, const float *Wp, const float *bias,
    float *out, unsigned int ldout, unsigned int M, unsigned int N, unsigned int K, int act)
{
    #pragma omp parallel for schedule(dynamic, 1)
    for (long n0 = 0; n0 < (long)N; n0 += COLS_PER_BLOCK)
    {
        unsigned int nb = (N - n0) < COLS_PER_BLOCK ? (unsigned int)(N - n0) : COLS_PER_BLOCK;
        for (unsigned int nn = 0; nn < nb; nn++)
            memset (out + (size_t)(n0 + nn) * ldout, 0, M * sizeof (float));
        oracle_sgemm_packed (M, nb, K, Wp, K, in + (size_t)n0 * ldin, ldin, out + (size_t)n0 * ldout, ldout);
        bias_act (out + (size_t)n0 * ldout, ldout, M, nb, bias, act);
    }
}

/* fully connected: K = IH*IW*IC in (h, w, c) order over the parent's NHWC image, one column per
   batch item (reference src/tiled_kernels.c:502-612; weight order src/apu.c:23-31).  The parent is
   given with its own ld, so the image is gathered into a dense K-vector first. */
void oracle_fc (const float *in, unsigned int ldin, const float *Wp, const float *bias,
    float *out, unsigned int ldout, unsigned int B, unsigned int IHW, unsigned int IC, unsigned int OC, int act)
{
    const unsigned int K = IHW * IC;
    float *dense = malloc ((size_t)B * K * sizeof (float));
    for (unsigned int b = 0; b < B; b++)
        for (unsigned int p = 0; p < IHW; p++)
            memcpy (dense + (size_t)b * K + (size_t)p * IC, in + ((size_t)b * IHW + p) * ldin, IC * sizeof (float));
    #pragma omp parallel for schedule(dynamic, 1)
    for (long m0 = 0; m0 < (long)OC; m0 += 64)
    {
        unsigned int mb = (OC - m0) < 64 ? (unsigned int)(OC - m0) : 64;
        for (unsigned int n = 0; n < B; n++)
            memset (out + (size_t)n * ldout + m0, 0, mb * sizeof (float));
        oracle_sgemm_packed (mb, B, K, Wp + (size_t)m0 * K, K, dense, K, out + m0, ldout);
        bias_act (out + m0, ldout, mb, B, bias ? bias + m0 : NULL, act);
    }
    free (dense);
}

/* max pooling, padding = -INF (reference src/tiled_kernels.c:411-455) */
void oracle_maxpool2d (const float *in, unsigned int ldin, float *out, unsigned int ldout,
    unsigned int B, unsigned int IH, unsigned int IW, unsigned int C,
    unsigned int KH, unsigned int KW, unsigned int stride, unsigned int pad, int act)
{
    const unsigned int OH = (IH + 2 * pad - (KH - 1) - 1) / stride + 1;
    const unsigned int OW = (IW + 2 * pad - (KW - 1) - 1) / stride + 1;
    #pragma omp parallel for
    for (long col = 0; col < (long)B * OH * OW; col++)
    {
        unsigned int b = col / (OH * OW), oh = (col % (OH * OW)) / OW, ow = col % OW;
        float *o = out + (size_t)col * ldout;
        for (unsigned int c = 0; c < C; c++) o[c] = -INFINITY;
        for (unsigned int kh = 0; kh < KH; kh++)
            for (unsigned int kw = 0; kw < KW; kw++)
            {
                int ih = (int)(oh * stride + kh) - (int)pad, iw = (int)(ow * stride + kw) - (int)pad;
                if (ih < 0 || ih >= (int)IH || iw < 0 || iw >= (int)IW) continue;
                const float *p = in + ((size_t)b * IH * IW + (size_t)ih * IW + iw) * ldin;
                for (unsigned int c = 0; c < C; c++) o[c] = o[c] >= p[c] ? o[c] : p[c];
            }
        oracle_activate (o, C, act);
    }
}

/* average pooling, divisor = KH*KW including padded taps (reference src/tiled_kernels.c:456-501) */
void oracle_avgpool2d (const float *in, unsigned int ldin, float *out, unsigned int ldout,
    unsigned int B, unsigned int IH, unsigned int IW, unsigned int C,
    unsigned int KH, unsigned int KW, unsigned int stride, unsigned int pad, int act)
{
    const unsigned int OH = (IH + 2 * pad - (KH - 1) - 1) / stride + 1;
    const unsigned int OW = (IW + 2 * pad - (KW - 1) - 1) / stride + 1;
    #pragma omp parallel for
    for (long col = 0; col < (long)B * OH * OW; col++)
    {
        unsigned int b = col / (OH * OW), oh = (col % (OH * OW)) / OW, ow = col % OW;
        float *o = out + (size_t)col * ldout;
        for (unsigned int c = 0; c < C; c++) o[c] = 0;
        for (unsigned int kh = 0; kh < KH; kh++)
            for (unsigned int kw = 0; kw < KW; kw++)
            {
                int ih = (int)(oh * stride + kh) - (int)pad, iw = (int)(ow * stride + kw) - (int)pad;
                if (ih < 0 || ih >= (int)IH || iw < 0 || iw >= (int)IW) continue;
                const float *p = in + ((size_t)b * IH * IW + (size_t)ih * IW + iw) * ldin;
                for (unsigned int c = 0; c < C; c++) o[c] += p[c];
            }
        for (unsigned int c = 0; c < C; c++) o[c] /= (KH * KW);
        oracle_activate (o, C, act);
    }
}

/* out = act(p0 + p1) (reference src/tiled_kernels.c:613-638) */
void oracle_residual (const float *p0, unsigned int ld0, const float *p1, unsigned int ld1,
    float *out, unsigned int ldout, unsigned int M, unsigned int N, int act)
{
    #pragma omp parallel for
    for (long n = 0; n < (long)N; n++)
    {
        float *o = out + (size_t)n * ldout;
        for (unsigned int m = 0; m < M; m++)
            o[m] = p0[(size_t)n * ld0 + m] + p1[(size_t)n * ld1 + m];
        oracle_activate (o, M, act);
    }
}

/* YOLO box decode (reference src/tiled_kernels.c:675-708).  Output column = (batch, anchor a, h, w),
   rows = classes + 5; reads channel a * rows + j of input column (batch, h, w):
   x, y = (sigmoid + cell index) * stride; w, h = exp * anchor size; the rest = sigmoid. */
void oracle_yolo (const float *in, unsigned int ldin, float *out, unsigned int ldout, const float *anchors,
    unsigned int B, unsigned int IH, unsigned int IW, unsigned int IC, unsigned int rows, unsigned int stride)
{
    const unsigned int A = IC / rows;
    for (unsigned int n = 0; n < B * IH * IW * A; n++)
    {
        const unsigned int b = n / (IH * IW * A), rem = n % (IH * IW * A), a = rem / (IH * IW), hw = rem % (IH * IW);
        const unsigned int h = hw / IW, w = hw % IW;
        const float *x = in + (size_t)((b * IH + h) * IW + w) * ldin + a * rows;
        float *o = out + (size_t)n * ldout;
        o[0] = (1.0f / (1.0f + expf (-x[0])) + w) * stride;
        o[1] = (1.0f / (1.0f + expf (-x[1])) + h) * stride;
        o[2] = expf (x[2]) * anchors[2 * a];
        o[3] = expf (x[3]) * anchors[2 * a + 1];
        for (unsigned int j = 4; j < rows; j++) o[j] = 1.0f / (1.0f + expf (-x[j]));
    }
}

/* nearest-neighbour upsampling of p0 by `stride`, concatenated along the channels with p1 at the
   output resolution (reference src/tiled_kernels.c:710-741) */
void oracle_append (const float *p0, unsigned int ld0, const float *p1, unsigned int ld1, float *out, unsigned int ldout,
    unsigned int B, unsigned int OH, unsigned int OW, unsigned int C0, unsigned int C1, unsigned int stride)
{
    const unsigned int IW = OW / stride, IH = OH / stride;
    for (unsigned int n = 0; n < B * OH * OW; n++)
    {
        const unsigned int b = n / (OH * OW), oh = (n / OW) % OH, ow = n % OW;
        const float *a = p0 + (size_t)((b * IH + oh / stride) * IW + ow / stride) * ld0;
        const float *c = p1 + (size_t)n * ld1;
        float *o = out + (size_t)n * ldout;
        memcpy (o, a, C0 * sizeof (float));
        memcpy (o + C0, c, C1 * sizeof (float));
    }
}

/* max-subtracted softmax over rows of each column (reference src/tiled_kernels.c:640-673) */
void oracle_softmax (const float *in, unsigned int ldin, float *out, unsigned int ldout, unsigned int M, unsigned int N)
{
    for (unsigned int n = 0; n < N; n++)
    {
        const float *x = in + (size_t)n * ldin;
        float *o = out + (size_t)n * ldout;
        float mx = x[0], sum = 0;
        for (unsigned int m = 1; m < M; m++) mx = mx >= x[m] ? mx : x[m];
        for (unsigned int m = 0; m < M; m++) { o[m] = expf (x[m] - mx); sum += o[m]; }
        for (unsigned int m = 0; m < M; m++) o[m] /= sum;
    }
}

/* single-pass mean / E[x^2] layernorm, eps 1e-6f (reference src/tiled_kernels.c:743-783) */
void oracle_layernorm (const float *in, unsigned int ldin, const float *weight, const float *bias,
    float *out, unsigned int ldout, unsigned int M, unsigned int N)
{
    #pragma omp parallel for
    for (long n = 0; n < (long)N; n++)
    {
        const float *x = in + (size_t)n * ldin;
        float *o = out + (size_t)n * ldout;
        float mean = 0, var = 0;
        for (unsigned int m = 0; m < M; m++) { mean += x[m]; var += x[m] * x[m]; }
        mean /= M; var /= M; var -= mean * mean;
        var = 1 / sqrtf (var + 1e-6f);
        for (unsigned int m = 0; m < M; m++)
        {
            o[m] = (x[m] - mean) * var * weight[m];
            if (bias != NULL) o[m] += bias[m];
        }
    }
}

/* scores = K.Q per (batch, head); causal mask writes -1e10 where key > query BEFORE the
   1/sqrt(hd) scale; exp without max subtraction; normalise (reference src/tiled_kernels.c:784-932).
   q, k: [B*S] columns (ldq / ldk), feature h*hd + j.  out: [B*H*S] columns of ldout, rows = key index. */
void oracle_k_attention (const float *q, unsigned int ldq, const float *k, unsigned int ldk,
    float *out, unsigned int ldout, unsigned int B, unsigned int H, unsigned int S, unsigned int hd, int masked)
{
    #pragma omp parallel for
    for (long col = 0; col < (long)B * H * S; col++)
    {
        unsigned int b = col / (H * S), h = (col % (H * S)) / S, n = col % S;
        const float *qv = q + ((size_t)b * S + n) * ldq + h * hd;
        float *o = out + (size_t)col * ldout;
        float total = 0;
        for (unsigned int m = 0; m < S; m++)
        {
            const float *kv = k + ((size_t)b * S + m) * ldk + h * hd;
            float acc = 0;
            for (unsigned int j = 0; j < hd; j++) acc += kv[j] * qv[j];
            if (masked && m > n) acc = -1e10;
            acc /= sqrtf (hd);
            o[m] = expf (acc);
            total += o[m];
        }
        for (unsigned int m = 0; m < S; m++) o[m] /= total;
    }
}

/* out[b,q, h*hd + j] = sum_s V[b,s,h*hd + j] * P[b,h,q,s] (reference src/tiled_kernels.c:934-1037) */
void oracle_v_attention (const float *p, unsigned int ldp, const float *v, unsigned int ldv,
    float *out, unsigned int ldout, unsigned int B, unsigned int H, unsigned int S, unsigned int hd)
{
    #pragma omp parallel for
    for (long col = 0; col < (long)B * S; col++)
    {
        unsigned int b = col / S, n = col % S;
        float *o = out + (size_t)col * ldout;
        for (unsigned int h = 0; h < H; h++)
        {
            const float *pv = p + (((size_t)b * H + h) * S + n) * ldp;
            for (unsigned int j = 0; j < hd; j++) o[h * hd + j] = 0;
            for (unsigned int s = 0; s < S; s++)
            {
                const float *vv = v + ((size_t)b * S + s) * ldv + h * hd;
                for (unsigned int j = 0; j < hd; j++) o[h * hd + j] += vv[j] * pv[s];
            }
        }
    }
}
