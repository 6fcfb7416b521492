/*
 * ckq_synth.c - seeded synthetic data and GGUF-format weight encoders.
 *
 * Host-only C.  The reference engine ships no Q5_K/Q6_K weight quantizer and
 * its Python Q4_K quantizer (scripts/q4_k_quantize.py:70-131) writes a byte
 * layout its own C kernels do not read, so the weights for the benchmark
 * shapes are produced here: fp32 ~N(mean,std) from a counter-based generator,
 * then simple min/max K-quant encoders that emit format-valid blocks with a
 * non-zero dmin.  A second mode writes "random valid blocks" (uniform bytes
 * for quants and packed scales, d in [0.01,0.1], dmin in [0.001,0.05]) as the
 * reference's own kernel tests do
 * (unittest/test_gemv_kernels_comprehensive.py:187-267).
 *
 * Everything is a pure function of (seed, index), so the CPU box and the GPU
 * box generate identical bytes.
 */
#include "ckq_synth.h"

#include <math.h>
#include <string.h>

/* ---- counter-based RNG: splitmix64 of (seed, index) ---------------------- */
static inline uint64_t mix64(uint64_t z)
{
    z += 0x9e3779b97f4a7c15ull;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

static inline uint64_t rnd_u64(uint64_t seed, uint64_t idx)
{
    return mix64(mix64(seed) ^ (idx * 0xd1342543de82ef95ull + 1));
}

/* uniform in (0,1], 53 bits */
static inline double rnd_unit(uint64_t seed, uint64_t idx)
{
    return ((double)(rnd_u64(seed, idx) >> 11) + 1.0) * (1.0 / 9007199254740992.0);
}

void ckq_synth_normal(float *out, size_t n, float mean, float std, uint64_t seed)
{
    /* Box-Muller on pairs (2i, 2i+1) */
    for (size_t i = 0; i < n; i += 2) {
        const double u1 = rnd_unit(seed, i), u2 = rnd_unit(seed, i + 1);
        const double r = sqrt(-2.0 * log(u1)), t = 6.283185307179586476925 * u2;
        out[i] = (float)(mean + std * r * cos(t));
        if (i + 1 < n) out[i + 1] = (float)(mean + std * r * sin(t));
    }
}

void ckq_synth_uniform(float *out, size_t n, float lo, float hi, uint64_t seed)
{
    for (size_t i = 0; i < n; ++i) out[i] = (float)(lo + (hi - lo) * rnd_unit(seed, i));
}

void ckq_synth_bytes(uint8_t *out, size_t n, uint64_t seed)
{
    size_t i = 0;
    for (; i + 8 <= n; i += 8) {
        const uint64_t v = rnd_u64(seed, i >> 3);
        memcpy(out + i, &v, 8);
    }
    if (i < n) {
        const uint64_t v = rnd_u64(seed, i >> 3);
        memcpy(out + i, &v, n - i);
    }
}

/* ---- fp16 ---------------------------------------------------------------- */
uint16_t ckq_synth_fp32_to_fp16(float f)
{
    /* round-to-nearest-even via double scaling; handles subnormals */
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    const float a = fabsf(f);
    if (a != a) return (uint16_t)(sign | 0x7e00u);
    if (a >= 65520.0f) return (uint16_t)(sign | 0x7c00u);
    if (a < 6.103515625e-05f) { /* subnormal half: multiples of 2^-24 */
        const float q = nearbyintf(a * 16777216.0f);
        return (uint16_t)(sign | (uint16_t)q);
    }
    int e;
    const float m = frexpf(a, &e);                    /* a = m * 2^e, m in [0.5,1) */
    float q = nearbyintf(m * 2048.0f);                /* 11-bit significand */
    if (q == 2048.0f) { q = 1024.0f; e += 1; }
    const int he = e + 14;                            /* biased half exponent */
    if (he >= 31) return (uint16_t)(sign | 0x7c00u);
    return (uint16_t)(sign | (uint16_t)(he << 10) | ((uint16_t)q & 0x3ffu));
}

float ckq_synth_fp16_to_fp32(uint16_t h)
{
    const int s = h >> 15, e = (h >> 10) & 31, m = h & 0x3ff;
    float v;
    if (e == 0) v = ldexpf((float)m, -24);
    else if (e == 31) v = m ? NAN : INFINITY;
    else v = ldexpf((float)(m | 0x400), e - 25);
    return s ? -v : v;
}

/* ---- 6-bit scale/min packing (layout read by ckernel_quant.h:227-251) ---- */
static void pack_scales_k4(const uint8_t sc[8], const uint8_t mn[8], uint8_t out[12])
{
    for (int j = 0; j < 4; ++j) {
        out[j]     = (uint8_t)((sc[j] & 63) | ((sc[j + 4] >> 4) << 6));
        out[j + 4] = (uint8_t)((mn[j] & 63) | ((mn[j + 4] >> 4) << 6));
        out[j + 8] = (uint8_t)((sc[j + 4] & 0x0f) | ((mn[j + 4] & 0x0f) << 4));
    }
}

static inline int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* Shared Q4_K / Q5_K encoder: w ~ d*sc*q - dmin*m, q in [0,qmax]. */
static void encode_k45(const float *w, int qmax, ckq_half *d_out, ckq_half *dmin_out,
                       uint8_t scales12[12], uint8_t q[256])
{
    float sub_scale[8], sub_min[8], max_scale = 0.0f, max_min = 0.0f;
    for (int j = 0; j < 8; ++j) {
        float lo = 0.0f, hi = 0.0f; /* range always contains 0 so that m >= 0 */
        for (int l = 0; l < 32; ++l) {
            const float v = w[32 * j + l];
            if (v < lo) lo = v;
            if (v > hi) hi = v;
        }
        sub_scale[j] = (hi - lo) / (float)qmax;
        sub_min[j]   = -lo;
        if (sub_scale[j] > max_scale) max_scale = sub_scale[j];
        if (sub_min[j] > max_min) max_min = sub_min[j];
    }
    const ckq_half hd = ckq_synth_fp32_to_fp16(max_scale / 63.0f);
    const ckq_half hm = ckq_synth_fp32_to_fp16(max_min / 63.0f);
    const float d = ckq_synth_fp16_to_fp32(hd), dmin = ckq_synth_fp16_to_fp32(hm);
    uint8_t sc[8], mn[8];
    for (int j = 0; j < 8; ++j) {
        sc[j] = (uint8_t)clampi(d > 0.0f ? (int)nearbyintf(sub_scale[j] / d) : 0, 0, 63);
        mn[j] = (uint8_t)clampi(dmin > 0.0f ? (int)nearbyintf(sub_min[j] / dmin) : 0, 0, 63);
        const float step = d * (float)sc[j], off = dmin * (float)mn[j];
        for (int l = 0; l < 32; ++l) {
            const int v = step > 0.0f ? (int)nearbyintf((w[32 * j + l] + off) / step) : 0;
            q[32 * j + l] = (uint8_t)clampi(v, 0, qmax);
        }
    }
    pack_scales_k4(sc, mn, scales12);
    *d_out = hd;
    *dmin_out = hm;
}

void ckq_synth_quantize_q4_k(const float *w, void *out, size_t n)
{
    ckq_block_q4_K *b = (ckq_block_q4_K *)out;
    for (size_t i = 0; i < n / CKQ_QK_K; ++i, w += CKQ_QK_K) {
        uint8_t q[256];
        encode_k45(w, 15, &b[i].d, &b[i].dmin, b[i].scales, q);
        for (int g = 0; g < 4; ++g)
            for (int l = 0; l < 32; ++l)
                b[i].qs[32 * g + l] = (uint8_t)(q[64 * g + l] | (q[64 * g + 32 + l] << 4));
    }
}

void ckq_synth_quantize_q5_k(const float *w, void *out, size_t n)
{
    ckq_block_q5_K *b = (ckq_block_q5_K *)out;
    for (size_t i = 0; i < n / CKQ_QK_K; ++i, w += CKQ_QK_K) {
        uint8_t q[256];
        encode_k45(w, 31, &b[i].d, &b[i].dmin, b[i].scales, q);
        memset(b[i].qh, 0, sizeof(b[i].qh));
        for (int g = 0; g < 4; ++g)
            for (int l = 0; l < 32; ++l) {
                const uint8_t lo = q[64 * g + l], hi = q[64 * g + 32 + l];
                b[i].qs[32 * g + l] = (uint8_t)((lo & 15) | ((hi & 15) << 4));
                b[i].qh[l] |= (uint8_t)(((lo >> 4) << (2 * g)) | ((hi >> 4) << (2 * g + 1)));
            }
    }
}

/* Q6_K: w ~ d*scale[e/16]*(q-32), q in [0,63]. */
void ckq_synth_quantize_q6_k(const float *w, void *out, size_t n)
{
    ckq_block_q6_K *b = (ckq_block_q6_K *)out;
    for (size_t i = 0; i < n / CKQ_QK_K; ++i, w += CKQ_QK_K) {
        float sub[16], amax_all = 0.0f;
        for (int j = 0; j < 16; ++j) {
            float amax = 0.0f;
            for (int l = 0; l < 16; ++l) {
                const float a = fabsf(w[16 * j + l]);
                if (a > amax) amax = a;
            }
            sub[j] = amax / 31.0f;
            if (sub[j] > amax_all) amax_all = sub[j];
        }
        const ckq_half hd = ckq_synth_fp32_to_fp16(amax_all / 127.0f);
        const float d = ckq_synth_fp16_to_fp32(hd);
        uint8_t q[256];
        for (int j = 0; j < 16; ++j) {
            const int s = clampi(d > 0.0f ? (int)nearbyintf(sub[j] / d) : 0, 0, 127);
            b[i].scales[j] = (int8_t)s;
            const float step = d * (float)s;
            for (int l = 0; l < 16; ++l) {
                const int v = step > 0.0f ? (int)nearbyintf(w[16 * j + l] / step) : 0;
                q[16 * j + l] = (uint8_t)(clampi(v, -32, 31) + 32);
            }
        }
        for (int h = 0; h < 2; ++h)
            for (int l = 0; l < 32; ++l) {
                const uint8_t q1 = q[128 * h + l], q2 = q[128 * h + 32 + l];
                const uint8_t q3 = q[128 * h + 64 + l], q4 = q[128 * h + 96 + l];
                b[i].ql[64 * h + l]      = (uint8_t)((q1 & 15) | ((q3 & 15) << 4));
                b[i].ql[64 * h + 32 + l] = (uint8_t)((q2 & 15) | ((q4 & 15) << 4));
                b[i].qh[32 * h + l] = (uint8_t)((q1 >> 4) | ((q2 >> 4) << 2) | ((q3 >> 4) << 4) | ((q4 >> 4) << 6));
            }
        b[i].d = hd;
    }
}

/* Q8_0 weights: d = amax/127 (fp16), q = round(w * 127/amax). */
void ckq_synth_quantize_q8_0(const float *w, void *out, size_t n)
{
    ckq_block_q8_0 *b = (ckq_block_q8_0 *)out;
    for (size_t i = 0; i < n / CKQ_QK8_0; ++i, w += CKQ_QK8_0) {
        float amax = 0.0f;
        for (int l = 0; l < 32; ++l) {
            const float a = fabsf(w[l]);
            if (a > amax) amax = a;
        }
        const float id = amax != 0.0f ? 127.0f / amax : 0.0f;
        b[i].d = ckq_synth_fp32_to_fp16(amax / 127.0f);
        for (int l = 0; l < 32; ++l) b[i].qs[l] = (int8_t)clampi((int)nearbyintf(w[l] * id), -127, 127);
    }
}

/* Q5_0 weights: d = (value of largest magnitude) / -16 (fp16), q = min(31, trunc(w/d + 16.5)). */
void ckq_synth_quantize_q5_0(const float *w, void *out, size_t n)
{
    ckq_block_q5_0 *b = (ckq_block_q5_0 *)out;
    for (size_t i = 0; i < n / CKQ_QK8_0; ++i, w += CKQ_QK8_0) {
        float amax = 0.0f, vmax = 0.0f;
        for (int l = 0; l < 32; ++l) {
            const float a = fabsf(w[l]);
            if (a > amax) { amax = a; vmax = w[l]; }
        }
        const float d = vmax / -16.0f, id = d != 0.0f ? 1.0f / d : 0.0f;
        uint32_t qh = 0;
        b[i].d = ckq_synth_fp32_to_fp16(d);
        for (int l = 0; l < 16; ++l) {
            const int q0 = clampi((int)(w[l] * id + 16.5f), 0, 31), q1 = clampi((int)(w[16 + l] * id + 16.5f), 0, 31);
            b[i].qs[l] = (uint8_t)((q0 & 15) | ((q1 & 15) << 4));
            qh |= (uint32_t)(q0 >> 4) << l;
            qh |= (uint32_t)(q1 >> 4) << (16 + l);
        }
        memcpy(b[i].qh, &qh, 4);
    }
}

int ckq_synth_quantize(int fmt, const float *w, void *out, size_t n)
{
    switch (fmt) {
    case CKQ_FMT_Q4_K: ckq_synth_quantize_q4_k(w, out, n); return 0;
    case CKQ_FMT_Q5_K: ckq_synth_quantize_q5_k(w, out, n); return 0;
    case CKQ_FMT_Q6_K: ckq_synth_quantize_q6_k(w, out, n); return 0;
    case CKQ_FMT_Q8_0: ckq_synth_quantize_q8_0(w, out, n); return 0;
    case CKQ_FMT_Q5_0: ckq_synth_quantize_q5_0(w, out, n); return 0;
    default: return -1;
    }
}

/* Weight matrix [rows x k] of N(mean,std) values quantized block by block
 * without materialising the fp32 matrix. */
int ckq_synth_weights(int fmt, void *out, int rows, int k, float mean, float std, uint64_t seed)
{
    const int be = ckq_block_elems(fmt);
    const size_t bb = ckq_block_bytes(fmt);
    if (bb == 0 || fmt == CKQ_FMT_Q8_K || k % be) return -1;
    const size_t nblocks = (size_t)rows * (size_t)(k / be);
    float tmp[CKQ_QK_K];
    for (size_t i = 0; i < nblocks; ++i) {
        ckq_synth_normal(tmp, (size_t)be, mean, std, mix64(seed) + i);
        ckq_synth_quantize(fmt, tmp, (uint8_t *)out + i * bb, (size_t)be);
    }
    return 0;
}

/* Random valid blocks: every bit pattern of quants and packed scales occurs. */
int ckq_synth_random_blocks(int fmt, void *out, size_t nblocks, uint64_t seed)
{
    const size_t bb = ckq_block_bytes(fmt);
    if (bb == 0) return -1;
    uint8_t *p = (uint8_t *)out;
    ckq_synth_bytes(p, nblocks * bb, seed);
    for (size_t i = 0; i < nblocks; ++i) {
        const float d  = (float)(0.01 + 0.09 * rnd_unit(seed ^ 0x5bd1e995u, 2 * i));
        const float dm = (float)(0.001 + 0.049 * rnd_unit(seed ^ 0x5bd1e995u, 2 * i + 1));
        uint8_t *blk = p + i * bb;
        switch (fmt) {
        case CKQ_FMT_Q4_K:
            ((ckq_block_q4_K *)blk)->d = ckq_synth_fp32_to_fp16(d);
            ((ckq_block_q4_K *)blk)->dmin = ckq_synth_fp32_to_fp16(dm);
            break;
        case CKQ_FMT_Q5_K:
            ((ckq_block_q5_K *)blk)->d = ckq_synth_fp32_to_fp16(d);
            ((ckq_block_q5_K *)blk)->dmin = ckq_synth_fp32_to_fp16(dm);
            break;
        case CKQ_FMT_Q6_K: {
            ckq_block_q6_K *b = (ckq_block_q6_K *)blk;
            b->d = ckq_synth_fp32_to_fp16(d);
            for (int j = 0; j < 16; ++j)
                if (b->scales[j] == -128) b->scales[j] = -127;
            break;
        }
        case CKQ_FMT_Q8_0: {
            ckq_block_q8_0 *b = (ckq_block_q8_0 *)blk;
            b->d = ckq_synth_fp32_to_fp16(d);
            for (int j = 0; j < 32; ++j)
                if (b->qs[j] == -128) b->qs[j] = -127;
            break;
        }
        case CKQ_FMT_Q5_0:
            ((ckq_block_q5_0 *)blk)->d = ckq_synth_fp32_to_fp16(d);
            break;
        case CKQ_FMT_Q8_K: {
            ckq_block_q8_K *b = (ckq_block_q8_K *)blk;
            b->d = d;
            for (int j = 0; j < 16; ++j) {
                int s = 0;
                for (int t = 0; t < 16; ++t) s += b->qs[16 * j + t];
                b->bsums[j] = (int16_t)s;
            }
            break;
        }
        default: return -1;
        }
    }
    return 0;
}
