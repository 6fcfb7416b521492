/*
 * ckq_oracle.c - CPU oracle for the quantized dequant-dot matmul path.
 *
 * TEST INFRASTRUCTURE ONLY: linked by the test-suite, the smoke check and the
 * CPU-baseline leg of the benchmark; never by the GPU library.
 *
 * Plain scalar C.  Build with -ffp-contract=off so that every fp32 product is
 * rounded before it is added (the order written here is the order executed).
 * Integer parts (quantized values, sub-block dots, block sums) are exact by
 * construction; fp32 parts follow the operation order of the reference
 * routine cited at each function.
 */
#include "ckq_oracle.h"
#include "../include/ckq_blocks.h"

#include <limits.h>
#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

/* ------------------------------------------------------------------------ */
/* fp16                                                                      */
/* ------------------------------------------------------------------------ */

/* IEEE binary16 -> binary32, all classes (reference: ckernel_quant.h:265-294). */
float orc_fp16_to_fp32(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h >> 15) << 31;
    const int      e    = (h >> 10) & 0x1f;
    uint32_t       m    = h & 0x3ffu;
    uint32_t       bits;
    if (e == 0x1f) {
        bits = sign | 0x7f800000u | (m << 13);
    } else if (e != 0) {
        bits = sign | ((uint32_t)(e + 112) << 23) | (m << 13);
    } else if (m == 0) {
        bits = sign;
    } else {
        /* subnormal half: value = m * 2^-24, exactly representable */
        float v = (float)m * 5.9604644775390625e-8f;
        memcpy(&bits, &v, 4);
        bits |= sign;
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* binary32 -> binary16, round-to-nearest-even, overflow to infinity
 * (reference: ckernel_quant.h:311-336 soft path, :355-357 F16C path). */
uint16_t orc_fp32_to_fp16(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    const uint32_t ax   = x & 0x7fffffffu;
    if (ax > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);            /* NaN */
    if (ax >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);           /* >= 65536 or inf */
    if (ax < 0x33000000u) return sign;                                   /* < 2^-25 -> 0 */
    int      e = (int)(ax >> 23) - 127;                                  /* unbiased */
    uint32_t m = (ax & 0x7fffffu) | 0x800000u;                           /* 24-bit significand */
    int      shift;                                                      /* bits to drop */
    uint32_t he;
    if (e < -14) { shift = 13 + (-14 - e); he = 0; }                     /* half subnormal */
    else         { shift = 13;             he = (uint32_t)(e + 15); }
    uint32_t q   = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t hlf = 1u << (shift - 1);
    if (rem > hlf || (rem == hlf && (q & 1u))) q++;
    uint32_t out;
    if (he == 0) out = q;                        /* q may carry into exponent 1: correct */
    else         out = ((he - 1) << 10) + q;     /* q includes the implicit bit (0x400) */
    if (out >= 0x7c00u) out = 0x7c00u;
    return (uint16_t)(sign | out);
}

/* ------------------------------------------------------------------------ */
/* 6-bit scale/min unpack                                                    */
/* ------------------------------------------------------------------------ */

/* Byte form (reference: ckernel_quant.h:227-251). */
void orc_unpack_scales_k4(const uint8_t *s, uint8_t *sc, uint8_t *m)
{
    for (int j = 0; j < 4; ++j) {
        sc[j]     = s[j] & 63;
        m[j]      = s[j + 4] & 63;
        sc[j + 4] = (uint8_t)((s[j + 8] & 0x0f) | ((s[j] >> 6) << 4));
        m[j + 4]  = (uint8_t)((s[j + 8] >> 4) | ((s[j + 4] >> 6) << 4));
    }
}

/* Word form (reference: gemm_kernels_q5_k.c:131-170): three little-endian
 * words masked and recombined; must give the same sixteen values. */
void orc_unpack_scales_k4_kmask(const uint8_t *s, uint8_t *sc, uint8_t *m)
{
    uint32_t u[3];
    memcpy(u, s, 12);
    const uint32_t sc_lo = u[0] & 0x3f3f3f3fu;
    const uint32_t sc_hi = (u[2] & 0x0f0f0f0fu) | (((u[0] >> 6) & 0x03030303u) << 4);
    const uint32_t m_lo  = u[1] & 0x3f3f3f3fu;
    const uint32_t m_hi  = ((u[2] >> 4) & 0x0f0f0f0fu) | (((u[1] >> 6) & 0x03030303u) << 4);
    memcpy(sc, &sc_lo, 4);
    memcpy(sc + 4, &sc_hi, 4);
    memcpy(m, &m_lo, 4);
    memcpy(m + 4, &m_hi, 4);
}

/* ------------------------------------------------------------------------ */
/* Block decoders: expand one super-block to 256 small integers              */
/* ------------------------------------------------------------------------ */

/* Q4_K element order (reference: gemm_kernels_q4k_q8k.c:135-161). */
static void q4k_expand(const ckq_block_q4_K *w, uint8_t q[256])
{
    for (int g = 0; g < 4; ++g)
        for (int l = 0; l < 32; ++l) {
            q[64 * g + l]      = w->qs[32 * g + l] & 0x0f;
            q[64 * g + 32 + l] = w->qs[32 * g + l] >> 4;
        }
}

/* Q5_K element order (reference: gemm_kernels_q5_k.c:149-161). */
static void q5k_expand(const ckq_block_q5_K *w, uint8_t q[256])
{
    for (int g = 0; g < 4; ++g)
        for (int l = 0; l < 32; ++l) {
            const int b_lo = (w->qh[l] >> (2 * g)) & 1;
            const int b_hi = (w->qh[l] >> (2 * g + 1)) & 1;
            q[64 * g + l]      = (uint8_t)((w->qs[32 * g + l] & 0x0f) | (b_lo << 4));
            q[64 * g + 32 + l] = (uint8_t)((w->qs[32 * g + l] >> 4) | (b_hi << 4));
        }
}

/* Q6_K element order, already offset by -32 (reference:
 * gemm_kernels_q6k_q8k.c:86-116).  Scale index of element e is e/16. */
static void q6k_expand(const ckq_block_q6_K *w, int8_t q[256])
{
    for (int n = 0; n < 2; ++n) {
        const uint8_t *ql = w->ql + 64 * n;
        const uint8_t *qh = w->qh + 32 * n;
        for (int l = 0; l < 32; ++l) {
            q[128 * n + l]      = (int8_t)(((ql[l] & 0x0f)      | (((qh[l] >> 0) & 3) << 4)) - 32);
            q[128 * n + 32 + l] = (int8_t)(((ql[l + 32] & 0x0f) | (((qh[l] >> 2) & 3) << 4)) - 32);
            q[128 * n + 64 + l] = (int8_t)(((ql[l] >> 4)        | (((qh[l] >> 4) & 3) << 4)) - 32);
            q[128 * n + 96 + l] = (int8_t)(((ql[l + 32] >> 4)   | (((qh[l] >> 6) & 3) << 4)) - 32);
        }
    }
}

/* ------------------------------------------------------------------------ */
/* Activation quantizers                                                     */
/* ------------------------------------------------------------------------ */

/* x86 cvtps2dq followed by two saturating packs: the fp32 value is rounded to
 * nearest-even; NaN and values outside int32 become INT_MIN; then clamp to
 * int8 (reference: quantize_row_q8_k_sse.c:61-68). */
static int8_t rne_sat_i8(float p)
{
    int v;
    if (!(p >= -2147483648.0f && p < 2147483648.0f)) v = INT_MIN;
    else v = (int)nearbyintf(p);
    if (v > 127) v = 127;
    if (v < -128) v = -128;
    return (int8_t)v;
}

/* fp32 -> Q8_K.  The scale comes from the FIRST element with the largest
 * magnitude, sign kept; iscale = -127/max; each product iscale*x is rounded
 * to fp32 and then to the nearest-even integer (reference: the SSE routine
 * every x86 build dispatches to, quantize_row_q8_k_sse.c:22-82; contract
 * stated in gemm_kernels_q4k_q8k.c:53-103). */
void orc_quantize_row_q8_k(const float *x, void *vy, int k)
{
    if (!x || !vy || k <= 0) return;
    ckq_block_q8_K *y = (ckq_block_q8_K *)vy;
    const int nb = k / CKQ_QK_K;
    for (int i = 0; i < nb; ++i, x += CKQ_QK_K) {
        float max = 0.0f, amax = 0.0f;
        for (int j = 0; j < CKQ_QK_K; ++j) {
            const float ax = fabsf(x[j]);
            if (ax > amax) { amax = ax; max = x[j]; }
        }
        if (amax == 0.0f) {
            memset(&y[i], 0, sizeof(y[i]));
            continue;
        }
        const float iscale = -127.0f / max;
        for (int j = 0; j < CKQ_QK_K; ++j) {
            volatile float p = x[j] * iscale; /* rounded product, never fused */
            y[i].qs[j] = rne_sat_i8(p);
        }
        for (int j = 0; j < CKQ_QK_K / 16; ++j) {
            int s = 0;
            for (int t = 0; t < 16; ++t) s += y[i].qs[16 * j + t];
            y[i].bsums[j] = (int16_t)s;
        }
        y[i].d = 1.0f / iscale;
    }
}

/* Row loop with output stride nb*292 (reference: gemm_kernels_q8_0.c:221-239). */
void orc_quantize_batch_q8_k(const float *x, void *vy, int rows, int k)
{
    const size_t out_stride = (size_t)(k / CKQ_QK_K) * sizeof(ckq_block_q8_K);
    for (int r = 0; r < rows; ++r)
        orc_quantize_row_q8_k(x + (size_t)r * k, (uint8_t *)vy + r * out_stride, k);
}

/* fp32 -> Q8_0: amax over 32; d = amax/127 stored as fp16 (RNE);
 * id = amax ? 127/amax : 0; q = RNE(x*id) saturated to int8
 * (reference: gemm_kernels_q8_0.c:70-146, the AVX path x86 builds run). */
void orc_quantize_row_q8_0(const float *x, void *vy, int k)
{
    ckq_block_q8_0 *y = (ckq_block_q8_0 *)vy;
    const int nb = k / CKQ_QK8_0;
    for (int i = 0; i < nb; ++i, x += CKQ_QK8_0) {
        float amax = 0.0f;
        for (int j = 0; j < CKQ_QK8_0; ++j) {
            const float ax = fabsf(x[j]);
            if (ax > amax) amax = ax;
        }
        const float d  = amax / 127.0f;
        const float id = amax != 0.0f ? 127.0f / amax : 0.0f;
        y[i].d = orc_fp32_to_fp16(d);
        for (int j = 0; j < CKQ_QK8_0; ++j) {
            volatile float p = x[j] * id;
            y[i].qs[j] = rne_sat_i8(p);
        }
    }
}

void orc_quantize_batch_q8_0(const float *x, void *vy, int rows, int k)
{
    const size_t out_stride = (size_t)(k / CKQ_QK8_0) * sizeof(ckq_block_q8_0);
    for (int r = 0; r < rows; ++r)
        orc_quantize_row_q8_0(x + (size_t)r * k, (uint8_t *)vy + r * out_stride, k);
}

/* ------------------------------------------------------------------------ */
/* Dequantizers                                                              */
/* ------------------------------------------------------------------------ */

/* w = d*sc*q - dmin*m (reference: dequant_kernels.c:336-385). */
void orc_dequant_q4_k_row(const void *src, float *dst, size_t n)
{
    const ckq_block_q4_K *b = (const ckq_block_q4_K *)src;
    for (size_t i = 0; i < n / CKQ_QK_K; ++i, dst += CKQ_QK_K) {
        uint8_t q[256], sc[8], m[8];
        q4k_expand(&b[i], q);
        orc_unpack_scales_k4(b[i].scales, sc, m);
        const float d = orc_fp16_to_fp32(b[i].d), dmin = orc_fp16_to_fp32(b[i].dmin);
        for (int j = 0; j < 8; ++j) {
            const float dj = d * (float)sc[j], mj = dmin * (float)m[j];
            for (int l = 0; l < 32; ++l) dst[32 * j + l] = dj * (float)q[32 * j + l] - mj;
        }
    }
}

/* Same formula with 5-bit q (layout: gemm_kernels_q5_k.c:149-161; formula in
 * that file's header comment :28-30). */
void orc_dequant_q5_k_row(const void *src, float *dst, size_t n)
{
    const ckq_block_q5_K *b = (const ckq_block_q5_K *)src;
    for (size_t i = 0; i < n / CKQ_QK_K; ++i, dst += CKQ_QK_K) {
        uint8_t q[256], sc[8], m[8];
        q5k_expand(&b[i], q);
        orc_unpack_scales_k4(b[i].scales, sc, m);
        const float d = orc_fp16_to_fp32(b[i].d), dmin = orc_fp16_to_fp32(b[i].dmin);
        for (int j = 0; j < 8; ++j) {
            const float dj = d * (float)sc[j], mj = dmin * (float)m[j];
            for (int l = 0; l < 32; ++l) dst[32 * j + l] = dj * (float)q[32 * j + l] - mj;
        }
    }
}

/* w = d*scale[e/16]*(q-32) (reference: dequant_kernels.c:396-430). */
void orc_dequant_q6_k_row(const void *src, float *dst, size_t n)
{
    const ckq_block_q6_K *b = (const ckq_block_q6_K *)src;
    for (size_t i = 0; i < n / CKQ_QK_K; ++i, dst += CKQ_QK_K) {
        int8_t q[256];
        q6k_expand(&b[i], q);
        const float d = orc_fp16_to_fp32(b[i].d);
        for (int e = 0; e < 256; ++e) dst[e] = d * (float)b[i].scales[e / 16] * (float)q[e];
    }
}

void orc_dequant_q8_0_row(const void *src, float *dst, size_t n)
{
    const ckq_block_q8_0 *b = (const ckq_block_q8_0 *)src;
    for (size_t i = 0; i < n / CKQ_QK8_0; ++i) {
        const float d = orc_fp16_to_fp32(b[i].d);
        for (int j = 0; j < CKQ_QK8_0; ++j) dst[32 * i + j] = d * (float)b[i].qs[j];
    }
}

void orc_dequant_q8_k_row(const void *src, float *dst, size_t n)
{
    const ckq_block_q8_K *b = (const ckq_block_q8_K *)src;
    for (size_t i = 0; i < n / CKQ_QK_K; ++i)
        for (int j = 0; j < CKQ_QK_K; ++j) dst[256 * i + j] = b[i].d * (float)b[i].qs[j];
}

/* Quantized embedding lookup (reference: src/kernels/embedding_kernels.c:76-260):
 * out[t] = dequant(row id[t]) over aligned_embed_dim elements, + pos[t] over the
 * first embed_dim when asked, zero from embed_dim on; ids outside [0,vocab)
 * read row 0; rows t >= token_count (up to context_window) are zero. */
void orc_embedding_forward(int fmt, const int32_t *token_ids, int token_count, int vocab_size,
                           const void *token_embeddings, const float *pos_embeddings, float *output,
                           int embed_dim, int aligned_embed_dim, int context_window, int add_pos)
{
    if (!token_ids || !token_embeddings || !output) return;
    int tokens = token_count < 0 ? 0 : token_count;
    if (tokens > context_window) tokens = context_window;
    const size_t rb = ckq_row_bytes(fmt, (size_t)aligned_embed_dim);
    for (int t = 0; t < tokens; ++t) {
        int id = token_ids[t];
        if (id < 0 || id >= vocab_size) id = 0;
        const uint8_t *row = (const uint8_t *)token_embeddings + (size_t)id * rb;
        float *out = output + (size_t)t * aligned_embed_dim;
        if (fmt == CKQ_FMT_Q4_K) orc_dequant_q4_k_row(row, out, (size_t)aligned_embed_dim);
        else if (fmt == CKQ_FMT_Q6_K) orc_dequant_q6_k_row(row, out, (size_t)aligned_embed_dim);
        else orc_dequant_q8_0_row(row, out, (size_t)aligned_embed_dim);
        if (add_pos && pos_embeddings)
            for (int d = 0; d < embed_dim; ++d) out[d] += pos_embeddings[(size_t)t * aligned_embed_dim + d];
        for (int d = embed_dim; d < aligned_embed_dim; ++d) out[d] = 0.0f;
    }
    for (int t = tokens; t < context_window; ++t)
        memset(output + (size_t)t * aligned_embed_dim, 0, (size_t)aligned_embed_dim * sizeof(float));
}

/* ------------------------------------------------------------------------ */
/* Integer sub-block dots                                                    */
/* ------------------------------------------------------------------------ */

void orc_subdots_q4_k_q8_k(const void *w_row, const void *x_q8, int K, int32_t *out)
{
    const ckq_block_q4_K *w = (const ckq_block_q4_K *)w_row;
    const ckq_block_q8_K *x = (const ckq_block_q8_K *)x_q8;
    for (int i = 0; i < K / CKQ_QK_K; ++i) {
        uint8_t q[256];
        q4k_expand(&w[i], q);
        for (int j = 0; j < 8; ++j) {
            int32_t s = 0;
            for (int l = 0; l < 32; ++l) s += (int32_t)q[32 * j + l] * (int32_t)x[i].qs[32 * j + l];
            out[8 * i + j] = s;
        }
    }
}

void orc_subdots_q5_k_q8_k(const void *w_row, const void *x_q8, int K, int32_t *out)
{
    const ckq_block_q5_K *w = (const ckq_block_q5_K *)w_row;
    const ckq_block_q8_K *x = (const ckq_block_q8_K *)x_q8;
    for (int i = 0; i < K / CKQ_QK_K; ++i) {
        uint8_t q[256];
        q5k_expand(&w[i], q);
        for (int j = 0; j < 8; ++j) {
            int32_t s = 0;
            for (int l = 0; l < 32; ++l) s += (int32_t)q[32 * j + l] * (int32_t)x[i].qs[32 * j + l];
            out[8 * i + j] = s;
        }
    }
}

void orc_subdots_q6_k_q8_k(const void *w_row, const void *x_q8, int K, int32_t *out)
{
    const ckq_block_q6_K *w = (const ckq_block_q6_K *)w_row;
    const ckq_block_q8_K *x = (const ckq_block_q8_K *)x_q8;
    for (int i = 0; i < K / CKQ_QK_K; ++i) {
        int8_t q[256];
        q6k_expand(&w[i], q);
        for (int j = 0; j < 16; ++j) {
            int32_t s = 0;
            for (int l = 0; l < 16; ++l) s += (int32_t)q[16 * j + l] * (int32_t)x[i].qs[16 * j + l];
            out[16 * i + j] = s;
        }
    }
}

void orc_subdots_q8_0_q8_0(const void *w_row, const void *x_q8, int K, int32_t *out)
{
    const ckq_block_q8_0 *w = (const ckq_block_q8_0 *)w_row;
    const ckq_block_q8_0 *x = (const ckq_block_q8_0 *)x_q8;
    for (int i = 0; i < K / CKQ_QK8_0; ++i) {
        int32_t s = 0;
        for (int l = 0; l < 32; ++l) s += (int32_t)w[i].qs[l] * (int32_t)x[i].qs[l];
        out[i] = s;
    }
}

/* ------------------------------------------------------------------------ */
/* Row dots                                                                  */
/* ------------------------------------------------------------------------ */

/* Q4_K x Q8_K: per block d = fp16(w.d)*x.d, dmin = fp16(w.dmin)*x.d; per
 * 64-group, in this order: += d*sc[2g]*S_lo, -= dmin*m[2g]*B_lo,
 * += d*sc[2g+1]*S_hi, -= dmin*m[2g+1]*B_hi, where B_* are sums of two STORED
 * bsums (reference: gemm_kernels_q4k_q8k.c:121-181). */
static float dot_q4k(const ckq_block_q4_K *w, const ckq_block_q8_K *x, int nb)
{
    float sumf = 0.0f;
    for (int i = 0; i < nb; ++i) {
        uint8_t q[256], sc[8], m[8];
        q4k_expand(&w[i], q);
        orc_unpack_scales_k4(w[i].scales, sc, m);
        const float d    = orc_fp16_to_fp32(w[i].d) * x[i].d;
        const float dmin = orc_fp16_to_fp32(w[i].dmin) * x[i].d;
        for (int j = 0; j < 8; ++j) {
            int32_t s = 0;
            for (int l = 0; l < 32; ++l) s += (int32_t)q[32 * j + l] * (int32_t)x[i].qs[32 * j + l];
            const int32_t bs = (int32_t)x[i].bsums[2 * j] + (int32_t)x[i].bsums[2 * j + 1];
            sumf += d * (float)sc[j] * (float)s;
            sumf -= dmin * (float)m[j] * (float)bs;
        }
    }
    return sumf;
}

/* Q5_K x Q8_K: per block sumi = sum_j bsums[j]*m[j/2] (16 stored bsums),
 * doti = sum_j sc[j]*S_j, ret = (fp16(d)*x.d)*doti - (fp16(dmin)*x.d)*sumi;
 * row = running fp32 sum of ret (reference: gemm_kernels_q5_k.c:130-208,
 * 321-327). */
static float dot_q5k(const ckq_block_q5_K *w, const ckq_block_q8_K *x, int nb)
{
    float sum = 0.0f;
    for (int i = 0; i < nb; ++i) {
        uint8_t q[256], sc[8], m[8];
        q5k_expand(&w[i], q);
        orc_unpack_scales_k4_kmask(w[i].scales, sc, m);
        int32_t sumi = 0, doti = 0;
        for (int j = 0; j < 16; ++j) sumi += (int32_t)x[i].bsums[j] * (int32_t)m[j / 2];
        for (int j = 0; j < 8; ++j) {
            int32_t s = 0;
            for (int l = 0; l < 32; ++l) s += (int32_t)q[32 * j + l] * (int32_t)x[i].qs[32 * j + l];
            doti += (int32_t)sc[j] * s;
        }
        const float d    = orc_fp16_to_fp32(w[i].d) * x[i].d;
        const float dmin = orc_fp16_to_fp32(w[i].dmin) * x[i].d;
        sum += d * (float)doti - dmin * (float)sumi;
    }
    return sum;
}

/* Q6_K x Q8_K scalar form: every element adds d*sc*q*q8 in fp32, four
 * streams per l (reference: gemm_kernels_q6k_q8k.c:70-120). */
static float dot_q6k_elementwise(const ckq_block_q6_K *w, const ckq_block_q8_K *x, int nb)
{
    float sumf = 0.0f;
    for (int i = 0; i < nb; ++i) {
        int8_t q[256];
        q6k_expand(&w[i], q);
        const float d = orc_fp16_to_fp32(w[i].d) * x[i].d;
        for (int n = 0; n < 2; ++n)
            for (int l = 0; l < 32; ++l)
                for (int r = 0; r < 4; ++r) {
                    const int e = 128 * n + 32 * r + l;
                    sumf += d * (float)w[i].scales[e / 16] * (float)q[e] * (float)x[i].qs[e];
                }
    }
    return sumf;
}

/* Q6_K x Q8_K integer block form, as the AVX2/AVX-512 routines x86 builds
 * dispatch to: per block eight int32 lanes, lane t collecting
 * scale*(q-32)*q8 over elements whose position inside their 32-run is in
 * [4t,4t+3]; acc[t] = fma(d, (float)lane[t], acc[t]); final sum
 * ((a0+a4)+(a1+a5)) + ((a2+a6)+(a3+a7)).  The activation's stored bsums are
 * NOT read (reference: gemm_kernels_q6k_q8k.c:601-695). */
static float dot_q6k_lanes8(const ckq_block_q6_K *w, const ckq_block_q8_K *x, int nb)
{
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int i = 0; i < nb; ++i) {
        int8_t q[256];
        q6k_expand(&w[i], q);
        const float d = orc_fp16_to_fp32(w[i].d) * x[i].d;
        int32_t lane[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int e = 0; e < 256; ++e)
            lane[(e % 32) / 4] += (int32_t)w[i].scales[e / 16] * (int32_t)q[e] * (int32_t)x[i].qs[e];
        for (int t = 0; t < 8; ++t) acc[t] = fmaf(d, (float)lane[t], acc[t]);
    }
    const float s0 = acc[0] + acc[4], s1 = acc[1] + acc[5], s2 = acc[2] + acc[6], s3 = acc[3] + acc[7];
    return (s0 + s1) + (s2 + s3);
}

/* Q8_0 x Q8_0 scalar: sumf += sumi * (fp16(dw)*fp16(dx)) per 32-block
 * (reference: gemm_kernels_q8_0.c:968-989). */
static float dot_q80(const ckq_block_q8_0 *w, const ckq_block_q8_0 *x, int nb)
{
    float sumf = 0.0f;
    for (int i = 0; i < nb; ++i) {
        int32_t s = 0;
        for (int l = 0; l < 32; ++l) s += (int32_t)w[i].qs[l] * (int32_t)x[i].qs[l];
        sumf += (float)s * (orc_fp16_to_fp32(w[i].d) * orc_fp16_to_fp32(x[i].d));
    }
    return sumf;
}

/* Q8_0 x Q8_0 in the AVX2 routine's order: eight fp32 lanes, lane t holding
 * the dot of bytes [4t,4t+3] of each block, acc = fma(d, q, acc), then
 * ((a0+a4)+(a2+a6)) + ((a1+a5)+(a3+a7)) (reference: gemm_kernels_q8_0.c:845-889,
 * 1031-1058). */
static float dot_q80_lanes8(const ckq_block_q8_0 *w, const ckq_block_q8_0 *x, int nb)
{
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int i = 0; i < nb; ++i) {
        const float d = orc_fp16_to_fp32(w[i].d) * orc_fp16_to_fp32(x[i].d);
        for (int t = 0; t < 8; ++t) {
            int32_t s = 0;
            for (int l = 0; l < 4; ++l) s += (int32_t)w[i].qs[4 * t + l] * (int32_t)x[i].qs[4 * t + l];
            acc[t] = fmaf(d, (float)s, acc[t]);
        }
    }
    const float r0 = acc[0] + acc[4], r1 = acc[1] + acc[5], r2 = acc[2] + acc[6], r3 = acc[3] + acc[7];
    return (r0 + r2) + (r1 + r3);
}

/* ------------------------------------------------------------------------ */
/* GEMV                                                                      */
/* ------------------------------------------------------------------------ */

/* Row range of thread ith of nth (reference: gemm_kernels_q4k_q8k.c:226-231). */
static int row_range(int M, int ith, int nth, int *r0, int *r1)
{
    if (ith < 0 || nth <= 0 || ith >= nth) return 0;
    const int dr = (M + nth - 1) / nth;
    *r0 = dr * ith;
    *r1 = (*r0 + dr < M) ? *r0 + dr : M;
    return *r0 < M;
}

void orc_gemv_q4_k_q8_k(float *y, const void *W, const void *x_q8, int M, int K)
{
    if (!y || !W || !x_q8 || M <= 0 || K <= 0) return;
    const int nb = K / CKQ_QK_K;
    const ckq_block_q4_K *w = (const ckq_block_q4_K *)W;
    for (int r = 0; r < M; ++r) y[r] = dot_q4k(w + (size_t)r * nb, (const ckq_block_q8_K *)x_q8, nb);
}

void orc_gemv_q4_k_q8_k_parallel(float *y, const void *W, const void *x_q8, int M, int K, int ith, int nth)
{
    if (!y || !W || !x_q8 || M <= 0 || K <= 0) return;
    int r0, r1;
    if (!row_range(M, ith, nth, &r0, &r1)) return;
    const int nb = K / CKQ_QK_K;
    const ckq_block_q4_K *w = (const ckq_block_q4_K *)W;
    for (int r = r0; r < r1; ++r) y[r] = dot_q4k(w + (size_t)r * nb, (const ckq_block_q8_K *)x_q8, nb);
}

void orc_gemv_q5_k_q8_k(float *y, const void *W, const void *x_q8, int M, int K)
{
    if (!y || !W || !x_q8 || M <= 0 || K <= 0) return;
    if (K % CKQ_QK_K != 0) return; /* gemm_kernels_q5_k.c:313-315 */
    const int nb = K / CKQ_QK_K;
    const ckq_block_q5_K *w = (const ckq_block_q5_K *)W;
    for (int r = 0; r < M; ++r) y[r] = dot_q5k(w + (size_t)r * nb, (const ckq_block_q8_K *)x_q8, nb);
}

/* fp32-activation adapter: quantize x to Q8_K, then the Q8_K kernel.  Only
 * the K%256==0, K<=32768 branch is restated; the reference's other branch
 * reads a different bit layout (gemm_kernels_q5_k.c:211-246) and is not part
 * of the GGUF contract. */
void orc_gemv_q5_k(float *y, const void *W, const float *x, int M, int K)
{
    if (!y || !W || !x || M <= 0 || K <= 0) return;
    if (K % CKQ_QK_K != 0 || K / CKQ_QK_K > 128) return;
    ckq_block_q8_K xq[128];
    orc_quantize_row_q8_k(x, xq, K);
    orc_gemv_q5_k_q8_k(y, W, xq, M, K);
}

void orc_gemv_q6_k_q8_k_ref(float *y, const void *W, const void *x_q8, int M, int K)
{
    if (!y || !W || !x_q8 || M <= 0 || K <= 0) return;
    const int nb = K / CKQ_QK_K;
    const ckq_block_q6_K *w = (const ckq_block_q6_K *)W;
    for (int r = 0; r < M; ++r)
        y[r] = dot_q6k_elementwise(w + (size_t)r * nb, (const ckq_block_q8_K *)x_q8, nb);
}

void orc_gemv_q6_k_q8_k(float *y, const void *W, const void *x_q8, int M, int K)
{
    if (!y || !W || !x_q8 || M <= 0 || K <= 0) return;
    const int nb = K / CKQ_QK_K;
    const ckq_block_q6_K *w = (const ckq_block_q6_K *)W;
    for (int r = 0; r < M; ++r)
        y[r] = dot_q6k_lanes8(w + (size_t)r * nb, (const ckq_block_q8_K *)x_q8, nb);
}

void orc_gemv_q6_k_q8_k_parallel(float *y, const void *W, const void *x_q8, int M, int K, int ith, int nth)
{
    if (!y || !W || !x_q8 || M <= 0 || K <= 0) return;
    int r0, r1;
    if (!row_range(M, ith, nth, &r0, &r1)) return;
    const int nb = K / CKQ_QK_K;
    const ckq_block_q6_K *w = (const ckq_block_q6_K *)W;
    for (int r = r0; r < r1; ++r)
        y[r] = dot_q6k_lanes8(w + (size_t)r * nb, (const ckq_block_q8_K *)x_q8, nb);
}

void orc_vec_dot_q6_k_q8_k(int n, float *s, const void *vx, const void *vy)
{
    if (!s || !vx || !vy || n <= 0) return;
    *s = dot_q6k_lanes8((const ckq_block_q6_K *)vx, (const ckq_block_q8_K *)vy, n / CKQ_QK_K);
}

void orc_gemv_q8_0_q8_0(float *y, const void *W, const void *x_q8, int M, int K)
{
    const int nb = K / CKQ_QK8_0;
    const ckq_block_q8_0 *w = (const ckq_block_q8_0 *)W;
    for (int r = 0; r < M; ++r) y[r] = dot_q80(w + (size_t)r * nb, (const ckq_block_q8_0 *)x_q8, nb);
}

void orc_gemv_q8_0_q8_0_lanes8(float *y, const void *W, const void *x_q8, int M, int K)
{
    const int nb = K / CKQ_QK8_0;
    const ckq_block_q8_0 *w = (const ckq_block_q8_0 *)W;
    for (int r = 0; r < M; ++r) y[r] = dot_q80_lanes8(w + (size_t)r * nb, (const ckq_block_q8_0 *)x_q8, nb);
}

void orc_gemv_q8_0_q8_0_parallel(float *y, const void *W, const void *x_q8, int M, int K, int ith, int nth)
{
    if (!y || !W || !x_q8 || M <= 0 || K <= 0) return;
    int r0, r1;
    if (!row_range(M, ith, nth, &r0, &r1)) return;
    const int nb = K / CKQ_QK8_0;
    const ckq_block_q8_0 *w = (const ckq_block_q8_0 *)W;
    for (int r = r0; r < r1; ++r) y[r] = dot_q80(w + (size_t)r * nb, (const ckq_block_q8_0 *)x_q8, nb);
}

void orc_vec_dot_q8_0_q8_0(int n, float *s, const void *vx, const void *vy)
{
    *s = dot_q80((const ckq_block_q8_0 *)vx, (const ckq_block_q8_0 *)vy, n / CKQ_QK8_0);
}

/* Q8_0 weights, fp32 activations: sum += d*q*x per element
 * (reference: gemm_kernels_q8_0.c:254-277). */
void orc_gemv_q8_0(float *y, const void *W, const float *x, int M, int K)
{
    const int nb = K / CKQ_QK8_0;
    const ckq_block_q8_0 *w = (const ckq_block_q8_0 *)W;
    for (int r = 0; r < M; ++r) {
        float sum = 0.0f;
        for (int b = 0; b < nb; ++b) {
            const ckq_block_q8_0 *blk = &w[(size_t)r * nb + b];
            const float d = orc_fp16_to_fp32(blk->d);
            for (int i = 0; i < CKQ_QK8_0; ++i) sum += d * (float)blk->qs[i] * x[32 * b + i];
        }
        y[r] = sum;
    }
}

/* Q4_K weights, fp32 activations, no activation quantization:
 * sum += (d*sc*q - dmin*m) * x per element, left to right
 * (reference: gemm_kernels_q4k.c:53-101; gemv_q4_k at :285-297 dispatches to
 * SIMD variants of the same sum, which differ in summation order only). */
void orc_gemv_q4_k(float *y, const void *W, const float *x, int M, int K)
{
    if (!y || !W || !x || M <= 0 || K <= 0) return;
    const int nb = K / CKQ_QK_K;
    const ckq_block_q4_K *w = (const ckq_block_q4_K *)W;
    for (int r = 0; r < M; ++r) {
        float sum = 0.0f;
        for (int b = 0; b < nb; ++b) {
            const ckq_block_q4_K *blk = &w[(size_t)r * nb + b];
            const float d = orc_fp16_to_fp32(blk->d), dmin = orc_fp16_to_fp32(blk->dmin);
            uint8_t sc[8], m[8];
            orc_unpack_scales_k4(blk->scales, sc, m);
            for (int g = 0; g < 4; ++g) {
                const float d1 = d * (float)sc[2 * g], m1 = dmin * (float)m[2 * g];
                const float d2 = d * (float)sc[2 * g + 1], m2 = dmin * (float)m[2 * g + 1];
                const uint8_t *qs = blk->qs + 32 * g;
                const float *xp = x + (size_t)b * CKQ_QK_K + 64 * g;
                for (int l = 0; l < 32; ++l) sum += (d1 * (float)(qs[l] & 0x0F) - m1) * xp[l];
                for (int l = 0; l < 32; ++l) sum += (d2 * (float)(qs[l] >> 4) - m2) * xp[l + 32];
            }
        }
        y[r] = sum;
    }
}

/* Q6_K weights, fp32 activations: sum += (d*sc*q) * x, four streams per l
 * (reference: gemm_kernels_q6k.c:39-76, gemv_q6_k at :169-193). */
void orc_gemv_q6_k(float *y, const void *W, const float *x, int M, int K)
{
    if (!y || !W || !x || M <= 0 || K <= 0) return;
    const int nb = K / CKQ_QK_K;
    const ckq_block_q6_K *w = (const ckq_block_q6_K *)W;
    for (int r = 0; r < M; ++r) {
        float sum = 0.0f;
        for (int b = 0; b < nb; ++b) {
            const ckq_block_q6_K *blk = &w[(size_t)r * nb + b];
            const float d = orc_fp16_to_fp32(blk->d);
            const uint8_t *ql = blk->ql, *qh = blk->qh;
            const int8_t *sc = blk->scales;
            const float *xp = x + (size_t)b * CKQ_QK_K;
            for (int n = 0; n < CKQ_QK_K; n += 128) {
                for (int l = 0; l < 32; ++l) {
                    const int is = l / 16;
                    const int8_t q1 = (int8_t)((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
                    const int8_t q2 = (int8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
                    const int8_t q3 = (int8_t)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                    const int8_t q4 = (int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                    sum += (d * (float)sc[is + 0] * (float)q1) * xp[l];
                    sum += (d * (float)sc[is + 2] * (float)q2) * xp[l + 32];
                    sum += (d * (float)sc[is + 4] * (float)q3) * xp[l + 64];
                    sum += (d * (float)sc[is + 6] * (float)q4) * xp[l + 96];
                }
                xp += 128; ql += 64; qh += 32; sc += 8;
            }
        }
        y[r] = sum;
    }
}

/* ------------------------------------------------------------------------ */
/* Fused producer: RMSNorm -> Q8_K                                           */
/* ------------------------------------------------------------------------ */

/* Reference: src/kernels/fused/rmsnorm_q8_k_fused.c:54-142 as an x86 build with
 * FMA compiles it.  Per token: sum of squares in eight strided lanes (lane j
 * takes x[8i+j]; gcc contracts the add of the product into one FMA when the
 * build enables FMA, which every AVX2 host build does), lanes combined as
 * ((l0+l4)+(l1+l5)) + ((l2+l6)+(l3+l7)); rstd = 1/sqrtf(sum/D + eps); then per
 * 256-block: n = (x*rstd)*gamma (two roundings), scale from the largest
 * |n| (NOT the signed first-largest of quantize_row_q8_k): iscale = -127/max,
 * d = 1/iscale (negative), q = RNE(n*iscale) saturated to int8, bsums of 16.
 * `fma` = 0 restates a build without FMA (product rounded before the add). */
static void rmsnorm_q8_k_fused_impl(const float *input, const float *gamma, void *vy,
                                    int tokens, int d_model, int aligned_embed_dim, float eps, int fma)
{
    if (!input || !gamma || !vy || tokens <= 0 || d_model <= 0) return;
    const int D = d_model, nb = D / CKQ_QK_K;
    ckq_block_q8_K *y = (ckq_block_q8_K *)vy;
    for (int t = 0; t < tokens; ++t) {
        const float *x = input + (size_t)t * aligned_embed_dim;
        float lane[8] = {0};
        for (int d = 0; d < D; d += 8)
            for (int j = 0; j < 8; ++j) {
                if (fma) lane[j] = fmaf(x[d + j], x[d + j], lane[j]);
                else { volatile float p = x[d + j] * x[d + j]; lane[j] = lane[j] + p; }
            }
        const float s04 = lane[0] + lane[4], s15 = lane[1] + lane[5], s26 = lane[2] + lane[6], s37 = lane[3] + lane[7];
        const float sum_sq = (s04 + s15) + (s26 + s37);
        const float rstd = 1.0f / sqrtf(sum_sq / (float)D + eps);
        for (int b = 0; b < nb; ++b) {
            const float *xb = x + b * CKQ_QK_K, *gb = gamma + b * CKQ_QK_K;
            ckq_block_q8_K *o = &y[(size_t)t * nb + b];
            float n[CKQ_QK_K], amax = 0.0f;
            for (int i = 0; i < CKQ_QK_K; ++i) {
                volatile float u = xb[i] * rstd;
                n[i] = u * gb[i];
                const float a = fabsf(n[i]);
                if (a > amax) amax = a;              /* maxps: a NaN operand never replaces the running max */
            }
            if (amax == 0.0f) { memset(o, 0, sizeof(*o)); continue; }
            const float iscale = -127.0f / amax;
            o->d = 1.0f / iscale;
            for (int j = 0; j < CKQ_QK_K; j += 16) {
                int bs = 0;
                for (int i = 0; i < 16; ++i) {
                    volatile float p = n[j + i] * iscale;
                    const int q = rne_sat_i8(p);
                    o->qs[j + i] = (int8_t)q;
                    bs += q;
                }
                o->bsums[j / 16] = (int16_t)bs;
            }
        }
    }
}

void orc_rmsnorm_q8_k_fused(const float *input, const float *gamma, void *vy,
                            int tokens, int d_model, int aligned_embed_dim, float eps)
{
    rmsnorm_q8_k_fused_impl(input, gamma, vy, tokens, d_model, aligned_embed_dim, eps, 1);
}

void orc_rmsnorm_q8_k_fused_nofma(const float *input, const float *gamma, void *vy,
                                  int tokens, int d_model, int aligned_embed_dim, float eps)
{
    rmsnorm_q8_k_fused_impl(input, gamma, vy, tokens, d_model, aligned_embed_dim, eps, 0);
}

/* ------------------------------------------------------------------------ */
/* GEMM                                                                      */
/* ------------------------------------------------------------------------ */

static void add_bias(float *C, const float *bias, int M, int N)
{
    if (!bias) return;
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j) C[(size_t)i * N + j] += bias[j];
}

void orc_gemm_q4_k_q8_k(float *Y, const void *W, const void *X_q8, int M, int N, int K)
{
    if (!Y || !W || !X_q8 || M <= 0 || N <= 0 || K <= 0) return;
    const size_t xs = (size_t)(K / CKQ_QK_K) * sizeof(ckq_block_q8_K);
    for (int n = 0; n < N; ++n)
        orc_gemv_q4_k_q8_k(Y + (size_t)n * M, W, (const uint8_t *)X_q8 + n * xs, M, K);
}

void orc_gemm_nt_q4_k_q8_k(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K)
{
    if (!A_q8 || !B || !C || M <= 0 || N <= 0 || K <= 0) return;
    orc_gemm_q4_k_q8_k(C, B, A_q8, N, M, K);
    add_bias(C, bias, M, N);
}

/* Bias is added to the finished row sum inside the store
 * (reference: gemm_kernels_q5_k.c:348-358). */
void orc_gemm_nt_q5_k_q8_k(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K)
{
    if (!A_q8 || !B || !C || M <= 0 || N <= 0 || K <= 0) return;
    if (K % CKQ_QK_K != 0) return;
    const int nb = K / CKQ_QK_K;
    const ckq_block_q8_K *a = (const ckq_block_q8_K *)A_q8;
    const ckq_block_q5_K *w = (const ckq_block_q5_K *)B;
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n)
            C[(size_t)m * N + n] = dot_q5k(w + (size_t)n * nb, a + (size_t)m * nb, nb) + (bias ? bias[n] : 0.0f);
}

void orc_gemm_nt_q5_k(const float *A, const void *B, const float *bias, float *C, int M, int N, int K)
{
    if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0) return;
    if (K % CKQ_QK_K != 0 || K / CKQ_QK_K > 128) return;
    ckq_block_q8_K aq[128];
    for (int m = 0; m < M; ++m) {
        orc_quantize_row_q8_k(A + (size_t)m * K, aq, K);
        orc_gemm_nt_q5_k_q8_k(aq, B, bias, C + (size_t)m * N, 1, N, K);
    }
}

void orc_gemm_q6_k_q8_k(float *Y, const void *W, const void *X_q8, int M, int N, int K)
{
    if (!Y || !W || !X_q8 || M <= 0 || N <= 0 || K <= 0) return;
    const size_t xs = (size_t)(K / CKQ_QK_K) * sizeof(ckq_block_q8_K);
    for (int n = 0; n < N; ++n)
        orc_gemv_q6_k_q8_k(Y + (size_t)n * M, W, (const uint8_t *)X_q8 + n * xs, M, K);
}

void orc_gemm_nt_q6_k_q8_k(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K)
{
    if (!A_q8 || !B || !C || M <= 0 || N <= 0 || K <= 0) return;
    orc_gemm_q6_k_q8_k(C, B, A_q8, N, M, K);
    add_bias(C, bias, M, N);
}

/* sum += (da*db) * (float)sumi per block, bias added afterwards
 * (reference: gemm_batch_int8.c:87-120,582-610). */
void orc_gemm_nt_q8_0_q8_0(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K)
{
    const int nb = K / CKQ_QK8_0;
    const ckq_block_q8_0 *a = (const ckq_block_q8_0 *)A_q8;
    const ckq_block_q8_0 *w = (const ckq_block_q8_0 *)B;
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            float sum = 0.0f;
            for (int b = 0; b < nb; ++b) {
                const ckq_block_q8_0 *ab = &a[(size_t)m * nb + b], *wb = &w[(size_t)n * nb + b];
                const float d = orc_fp16_to_fp32(ab->d) * orc_fp16_to_fp32(wb->d);
                int32_t s = 0;
                for (int l = 0; l < 32; ++l) s += (int32_t)ab->qs[l] * (int32_t)wb->qs[l];
                sum += d * (float)s;
            }
            C[(size_t)m * N + n] = sum;
        }
    add_bias(C, bias, M, N);
}

/* ------------------------------------------------------------------------ */
/* Exact evaluation                                                          */
/* ------------------------------------------------------------------------ */

void orc_gemv_exact_f64(int fmt, double *y, const void *W, const void *x_q8, int M, int K)
{
    if (fmt == CKQ_FMT_Q8_0) {
        const int nb = K / CKQ_QK8_0;
        const ckq_block_q8_0 *w = (const ckq_block_q8_0 *)W, *x = (const ckq_block_q8_0 *)x_q8;
        for (int r = 0; r < M; ++r) {
            double acc = 0.0;
            for (int b = 0; b < nb; ++b) {
                int32_t s = 0;
                for (int l = 0; l < 32; ++l) s += (int32_t)w[(size_t)r * nb + b].qs[l] * (int32_t)x[b].qs[l];
                acc += (double)orc_fp16_to_fp32(w[(size_t)r * nb + b].d) * (double)orc_fp16_to_fp32(x[b].d) * (double)s;
            }
            y[r] = acc;
        }
        return;
    }
    const int nb = K / CKQ_QK_K;
    const ckq_block_q8_K *x = (const ckq_block_q8_K *)x_q8;
    for (int r = 0; r < M; ++r) {
        double acc = 0.0;
        for (int b = 0; b < nb; ++b) {
            int64_t i1 = 0, i2 = 0;
            double d = 0.0, dmin = 0.0;
            if (fmt == CKQ_FMT_Q4_K || fmt == CKQ_FMT_Q5_K) {
                uint8_t q[256], sc[8], m[8];
                if (fmt == CKQ_FMT_Q4_K) {
                    const ckq_block_q4_K *w = (const ckq_block_q4_K *)W + (size_t)r * nb + b;
                    q4k_expand(w, q);
                    orc_unpack_scales_k4(w->scales, sc, m);
                    d = orc_fp16_to_fp32(w->d);
                    dmin = orc_fp16_to_fp32(w->dmin);
                } else {
                    const ckq_block_q5_K *w = (const ckq_block_q5_K *)W + (size_t)r * nb + b;
                    q5k_expand(w, q);
                    orc_unpack_scales_k4(w->scales, sc, m);
                    d = orc_fp16_to_fp32(w->d);
                    dmin = orc_fp16_to_fp32(w->dmin);
                }
                for (int j = 0; j < 8; ++j) {
                    int32_t s = 0;
                    for (int l = 0; l < 32; ++l) s += (int32_t)q[32 * j + l] * (int32_t)x[b].qs[32 * j + l];
                    i1 += (int64_t)sc[j] * s;
                    i2 += (int64_t)m[j] * ((int32_t)x[b].bsums[2 * j] + (int32_t)x[b].bsums[2 * j + 1]);
                }
            } else { /* Q6_K */
                const ckq_block_q6_K *w = (const ckq_block_q6_K *)W + (size_t)r * nb + b;
                int8_t q[256];
                q6k_expand(w, q);
                d = orc_fp16_to_fp32(w->d);
                for (int e = 0; e < 256; ++e) i1 += (int64_t)w->scales[e / 16] * q[e] * x[b].qs[e];
            }
            acc += (double)x[b].d * (d * (double)i1 - dmin * (double)i2);
        }
        y[r] = acc;
    }
}

/* ------------------------------------------------------------------------ */
/* Threaded GEMV for the CPU baseline                                        */
/* ------------------------------------------------------------------------ */

typedef struct {
    int fmt, M, K, ith, nth;
    float *y;
    const void *W, *x;
} thr_arg;

static void *thr_main(void *p)
{
    thr_arg *a = (thr_arg *)p;
    switch (a->fmt) {
    case CKQ_FMT_Q4_K: orc_gemv_q4_k_q8_k_parallel(a->y, a->W, a->x, a->M, a->K, a->ith, a->nth); break;
    case CKQ_FMT_Q6_K: orc_gemv_q6_k_q8_k_parallel(a->y, a->W, a->x, a->M, a->K, a->ith, a->nth); break;
    case CKQ_FMT_Q8_0: orc_gemv_q8_0_q8_0_parallel(a->y, a->W, a->x, a->M, a->K, a->ith, a->nth); break;
    default: {
        int r0, r1;
        if (row_range(a->M, a->ith, a->nth, &r0, &r1)) {
            const size_t rb = ckq_row_bytes(CKQ_FMT_Q5_K, a->K);
            orc_gemv_q5_k_q8_k(a->y + r0, (const uint8_t *)a->W + r0 * rb, a->x, r1 - r0, a->K);
        }
    }
    }
    return NULL;
}

void orc_gemv_threads(int fmt, float *y, const void *W, const void *x_q8, int M, int K, int nth)
{
    if (nth < 1) nth = 1;
    if (nth > 256) nth = 256;
    pthread_t tid[256];
    thr_arg   arg[256];
    for (int t = 0; t < nth; ++t) {
        arg[t] = (thr_arg){fmt, M, K, t, nth, y, W, x_q8};
        if (t > 0) pthread_create(&tid[t], NULL, thr_main, &arg[t]);
    }
    thr_main(&arg[0]);
    for (int t = 1; t < nth; ++t) pthread_join(tid[t], NULL);
}

/* Timing harness for the CPU baseline: `nth` persistent threads (the caller is
 * thread 0) run fn(y, W, x, M, K, ith, nth) `iters` times, every round between
 * two barriers, as the reference's thread pool runs a split GEMV
 * (src/ck_threadpool.c:289-349: wake the workers, every thread takes its `ith`,
 * barrier).  seconds[i] is the wall time of round i as thread 0 sees it.  The
 * kernel is the caller's: the compiled reference's *_parallel_simd entry point,
 * or this file's restatement. */
typedef struct {
    pthread_mutex_t   mu;
    pthread_cond_t    cv;
    int               go;      /* 0 wait, 1 run, -1 give up (a thread could not be created) */
    pthread_barrier_t bar;
} time_gate;

typedef struct {
    orc_split_gemv_fn fn;
    float *y;
    const void *W, *x;
    int M, K, ith, nth, iters;
    time_gate *gate;
    size_t w_stride;           /* round i reads the weight copy at W + (i % w_copies) * w_stride */
    int    w_copies;
} time_arg;

static void *time_main(void *p)
{
    time_arg *a = (time_arg *)p;
    pthread_mutex_lock(&a->gate->mu);
    while (a->gate->go == 0) pthread_cond_wait(&a->gate->cv, &a->gate->mu);
    const int go = a->gate->go;
    pthread_mutex_unlock(&a->gate->mu);
    if (go < 0) return NULL;
    for (int i = 0; i < a->iters; ++i) {
        pthread_barrier_wait(&a->gate->bar);
        a->fn(a->y, (const uint8_t *)a->W + (size_t)(i % a->w_copies) * a->w_stride, a->x, a->M, a->K, a->ith, a->nth);
        pthread_barrier_wait(&a->gate->bar);
    }
    return NULL;
}

int orc_time_split_gemv(orc_split_gemv_fn fn, float *y, const void *W, const void *x_q8, int M, int K, int nth, int iters,
                        double *seconds)
{
    return orc_time_split_gemv_rotating(fn, y, W, 0, 1, x_q8, M, K, nth, iters, seconds);
}

/* The same with `w_copies` copies of the weights, `w_stride` bytes apart: round i
 * reads copy i % w_copies, so that with enough copies the weights come from DRAM
 * and not from the last-level cache. */
int orc_time_split_gemv_rotating(orc_split_gemv_fn fn, float *y, const void *W, size_t w_stride, int w_copies,
                                 const void *x_q8, int M, int K, int nth, int iters, double *seconds)
{
    if (!fn || !y || !W || !x_q8 || !seconds || M <= 0 || K <= 0 || nth < 1 || nth > 256 || iters < 1 || w_copies < 1) return -1;
    time_gate gate;
    if (pthread_barrier_init(&gate.bar, NULL, (unsigned)nth)) return -1;
    pthread_mutex_init(&gate.mu, NULL);
    pthread_cond_init(&gate.cv, NULL);
    gate.go = 0;
    pthread_t tid[256];
    time_arg  arg[256];
    int made = 1;
    for (; made < nth; ++made) {
        arg[made] = (time_arg){fn, y, W, x_q8, M, K, made, nth, iters, &gate, w_stride, w_copies};
        if (pthread_create(&tid[made], NULL, time_main, &arg[made])) break;
    }
    const int ok = made == nth;      /* a thread short: the barrier would never open, so nobody enters it */
    pthread_mutex_lock(&gate.mu);
    gate.go = ok ? 1 : -1;
    pthread_cond_broadcast(&gate.cv);
    pthread_mutex_unlock(&gate.mu);
    for (int i = 0; ok && i < iters; ++i) {
        struct timespec t0, t1;
        pthread_barrier_wait(&gate.bar);
        clock_gettime(CLOCK_MONOTONIC, &t0);
        fn(y, (const uint8_t *)W + (size_t)(i % w_copies) * w_stride, x_q8, M, K, 0, nth);
        pthread_barrier_wait(&gate.bar);
        clock_gettime(CLOCK_MONOTONIC, &t1);
        seconds[i] = (double)(t1.tv_sec - t0.tv_sec) + 1e-9 * (double)(t1.tv_nsec - t0.tv_nsec);
    }
    for (int t = 1; t < made; ++t) pthread_join(tid[t], NULL);
    pthread_barrier_destroy(&gate.bar);
    pthread_cond_destroy(&gate.cv);
    pthread_mutex_destroy(&gate.mu);
    return ok ? 0 : -1;
}

/* fp32-activation GEMMs: a token loop over the GEMV, then the bias
 * (reference: gemm_kernels_q4k.c:316-330,461-469,683-711; gemm_kernels_q6k.c:195-240;
 * gemm_kernels_q8_0.c:658-696). */
void orc_gemm_q4_k(float *Y, const void *W, const float *X, int M, int N, int K)
{
    if (!Y || !W || !X || M <= 0 || N <= 0 || K <= 0) return;
    for (int n = 0; n < N; ++n) orc_gemv_q4_k(Y + (size_t)n * M, W, X + (size_t)n * K, M, K);
}

void orc_gemm_nt_q4_k(const float *A, const void *B, const float *bias, float *C, int M, int N, int K)
{
    if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0) return;
    orc_gemm_q4_k(C, B, A, N, M, K);
    add_bias(C, bias, M, N);
}

void orc_gemm_q6_k(float *Y, const void *W, const float *X, int M, int N, int K)
{
    if (!Y || !W || !X || M <= 0 || N <= 0 || K <= 0) return;
    for (int n = 0; n < N; ++n) orc_gemv_q6_k(Y + (size_t)n * M, W, X + (size_t)n * K, M, K);
}

void orc_gemm_nt_q6_k(const float *A, const void *B, const float *bias, float *C, int M, int N, int K)
{
    if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0) return;
    orc_gemm_q6_k(C, B, A, N, M, K);
    add_bias(C, bias, M, N);
}

void orc_gemm_nt_q8_0(const float *A, const void *B, const float *bias, float *C, int M, int N, int K)
{
    if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0) return;
    for (int m = 0; m < M; ++m) orc_gemv_q8_0(C + (size_t)m * N, B, A + (size_t)m * K, N, K);
    add_bias(C, bias, M, N);
}


/* ------------------------------------------------------------------------ */
/* Q5_0 x Q8_0                                                               */
/* ------------------------------------------------------------------------ */

/* value index l of a Q5_0 block, already minus 16 (gemm_kernels_q5_0.c:917-927) */
static int q5_0_value(const ckq_block_q5_0 *b, int l)
{
    uint32_t qh;
    memcpy(&qh, b->qh, 4);
    const int nib = l < 16 ? (b->qs[l] & 0x0F) : (b->qs[l - 16] >> 4);
    return (nib | (int)(((qh >> l) & 1u) << 4)) - 16;
}

static int32_t q5_0_block_dot(const ckq_block_q5_0 *w, const ckq_block_q8_0 *x)
{
    int32_t s = 0;
    for (int l = 0; l < 32; ++l) s += (int32_t)q5_0_value(w, l) * (int32_t)x->qs[l];
    return s;
}

void orc_subdots_q5_0_q8_0(const void *w_row, const void *x_q8, int K, int32_t *out)
{
    const ckq_block_q5_0 *w = (const ckq_block_q5_0 *)w_row;
    const ckq_block_q8_0 *x = (const ckq_block_q8_0 *)x_q8;
    for (int i = 0; i < K / CKQ_QK8_0; ++i) out[i] = q5_0_block_dot(&w[i], &x[i]);
}

void orc_vec_dot_q5_0_q8_0(int n, float *s, const void *vx, const void *vy)
{
    const ckq_block_q5_0 *w = (const ckq_block_q5_0 *)vx;
    const ckq_block_q8_0 *x = (const ckq_block_q8_0 *)vy;
    /* the reference's x86 builds enable FMA, which fuses this multiply-add
     * (the golden test pins that choice bit for bit) */
    float sumf = 0.0f;
    for (int i = 0; i < n / CKQ_QK8_0; ++i)
        sumf = fmaf(orc_fp16_to_fp32(w[i].d) * orc_fp16_to_fp32(x[i].d), (float)q5_0_block_dot(&w[i], &x[i]), sumf);
    *s = sumf;
}

void orc_gemv_q5_0_q8_0(float *y, const void *W, const void *x_q8, int M, int K)
{
    if (!y || !W || !x_q8 || M <= 0 || K <= 0) return;
    const size_t rb = (size_t)(K / CKQ_QK8_0) * sizeof(ckq_block_q5_0);
    for (int r = 0; r < M; ++r) orc_vec_dot_q5_0_q8_0(K, &y[r], (const uint8_t *)W + (size_t)r * rb, x_q8);
}

void orc_gemm_nt_q5_0_q8_0(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K)
{
    if (!A_q8 || !B || !C || M <= 0 || N <= 0 || K <= 0) return;
    const size_t wb = (size_t)(K / CKQ_QK8_0) * sizeof(ckq_block_q5_0), xb = (size_t)(K / CKQ_QK8_0) * sizeof(ckq_block_q8_0);
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            float *out = &C[(size_t)m * N + n];
            orc_vec_dot_q5_0_q8_0(K, out, (const uint8_t *)B + (size_t)n * wb, (const uint8_t *)A_q8 + (size_t)m * xb);
            if (bias) *out += bias[n];
        }
}

void orc_q5_0_to_q8_0(const void *src, void *dst, size_t nblocks)
{
    const ckq_block_q5_0 *s = (const ckq_block_q5_0 *)src;
    ckq_block_q8_0 *d = (ckq_block_q8_0 *)dst;
    for (size_t i = 0; i < nblocks; ++i) {
        d[i].d = s[i].d;
        for (int l = 0; l < 32; ++l) d[i].qs[l] = (int8_t)q5_0_value(&s[i], l);
    }
}

/* ------------------------------------------------------------------------ */
/* Fused prefill MLP                                                         */
/* ------------------------------------------------------------------------ */

/* fused/prefill_fused_gemm.c:904-906 */
static float silu_prefill(float x) { return x / (1.0f + expf(-x)); }

/* The SwiGLU step and its quantization (fused/prefill_fused_gemm.c:1034-1047):
 * g = silu(g) * u element by element, then quantize_row_q8_k of each row. */
void orc_swiglu_q8_k(const float *gate, const float *up, void *y, int rows, int k, long ld)
{
    if (!gate || !up || !y || rows <= 0 || k <= 0 || k % 256) return;
    float *row = (float *)malloc((size_t)k * sizeof(float));
    if (!row) return;
    const size_t rb = (size_t)(k / 256) * sizeof(ckq_block_q8_K);
    for (int i = 0; i < rows; ++i) {
        const float *g = gate + (size_t)i * (size_t)ld, *u = up + (size_t)i * (size_t)ld;
        for (int j = 0; j < k; ++j) row[j] = silu_prefill(g[j]) * u[j];
        orc_quantize_row_q8_k(row, (uint8_t *)y + (size_t)i * rb, k);
    }
    free(row);
}

/* fused/prefill_fused_gemm.c:964-1060.  The reference walks the sequence in
 * tiles of 64 tokens; every step is row-wise, so the tiling does not change
 * any value and is not restated. */
void orc_fused_mlp_swiglu_prefill_w1w2_quant(const float *x, const void *W1, const float *B1, int w1_dt,
                                             const void *W2, const float *B2, int w2_dt, float *output,
                                             int seq_len, int embed_dim, int aligned_embed_dim,
                                             int intermediate_dim, int aligned_intermediate_dim,
                                             float *gate_up_out, void *h_q8k_out)
{
    enum { DT_Q4_K = 7, DT_Q6_K = 8, DT_Q8_0 = 9, DT_Q5_0 = 11 };
    if (!x || !W1 || !W2 || !output) return;
    if (seq_len <= 0 || embed_dim <= 0 || aligned_embed_dim <= 0 || intermediate_dim <= 0 ||
        aligned_intermediate_dim <= 0)
        return;
    if (aligned_embed_dim < embed_dim || aligned_intermediate_dim < intermediate_dim) return;
    if ((aligned_embed_dim % 32) != 0 || (aligned_intermediate_dim % 256) != 0) return;
    if ((w1_dt != DT_Q8_0 && w1_dt != DT_Q5_0) || (w2_dt != DT_Q4_K && w2_dt != DT_Q6_K)) return;

    const int E = aligned_embed_dim, I = aligned_intermediate_dim;
    const size_t q8_row = (size_t)(E / 32) * sizeof(ckq_block_q8_0);
    const size_t q8k_row = (size_t)(I / 256) * sizeof(ckq_block_q8_K);
    uint8_t *xq = (uint8_t *)malloc((size_t)seq_len * q8_row);
    float *gate = (float *)malloc((size_t)seq_len * I * sizeof(float));
    float *up = (float *)malloc((size_t)seq_len * I * sizeof(float));
    uint8_t *hq = (uint8_t *)malloc((size_t)seq_len * q8k_row);
    if (xq && gate && up && hq) {
        for (int t = 0; t < seq_len; ++t) orc_quantize_row_q8_0(x + (size_t)t * E, xq + (size_t)t * q8_row, E);
        const size_t w1_row = w1_dt == DT_Q8_0 ? q8_row : (size_t)(E / 32) * sizeof(ckq_block_q5_0);
        const uint8_t *w_gate = (const uint8_t *)W1, *w_up = w_gate + (size_t)I * w1_row;
        if (w1_dt == DT_Q8_0) {
            orc_gemm_nt_q8_0_q8_0(xq, w_gate, B1, gate, seq_len, I, E);
            orc_gemm_nt_q8_0_q8_0(xq, w_up, B1 ? B1 + I : NULL, up, seq_len, I, E);
        } else {
            orc_gemm_nt_q5_0_q8_0(xq, w_gate, B1, gate, seq_len, I, E);
            orc_gemm_nt_q5_0_q8_0(xq, w_up, B1 ? B1 + I : NULL, up, seq_len, I, E);
        }
        orc_swiglu_q8_k(gate, up, hq, seq_len, I, I);
        if (gate_up_out)
            for (int t = 0; t < seq_len; ++t) {
                for (int j = 0; j < I; ++j) gate_up_out[(size_t)t * 2 * I + j] = silu_prefill(gate[(size_t)t * I + j]) * up[(size_t)t * I + j];
                memcpy(gate_up_out + (size_t)t * 2 * I + I, up + (size_t)t * I, (size_t)I * sizeof(float));
            }
        if (h_q8k_out) memcpy(h_q8k_out, hq, (size_t)seq_len * q8k_row);
        if (w2_dt == DT_Q4_K) orc_gemm_nt_q4_k_q8_k(hq, W2, B2, output, seq_len, E, I);
        else                  orc_gemm_nt_q6_k_q8_k(hq, W2, B2, output, seq_len, E, I);
    }
    free(xq); free(gate); free(up); free(hq);
}
