/*
 * asan_harness.c - CPU sanitizer pass (test infrastructure, like the rest of
 * oracle/): drives the oracle, the synthetic-data encoders and the library's
 * HIP-free host helpers under AddressSanitizer and UndefinedBehaviorSanitizer.
 * Every buffer is a heap allocation of exactly the size the callee may touch,
 * so an access one byte out of range is a report; shapes are ragged on
 * purpose (one block, odd row counts, row ranges that leave threads idle).
 * The reference has sanitizer targets of its own for its kernels
 * (Makefile:2408, version/v7/scripts/ck_run_v7.py:4512); this is the
 * counterpart for the code of this repository that runs on the CPU.
 *
 *   make -C oracle asan && oracle/asan_harness      (exit status 0, no report)
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "ckq_blocks.h"
#include "ckq_oracle.h"
#include "ckq_pure.h"
#include "ckq_synth.h"

static int failures = 0;
#define CHECK(cond)                                                                  \
    do {                                                                             \
        if (!(cond)) { fprintf(stderr, "asan_harness: %s:%d: %s\n", __FILE__, __LINE__, #cond); ++failures; } \
    } while (0)

static size_t row_bytes(int fmt, int k)
{
    switch (fmt) {
    case CKQ_FMT_Q4_K: return (size_t)(k / 256) * 144;
    case CKQ_FMT_Q5_K: return (size_t)(k / 256) * 176;
    case CKQ_FMT_Q6_K: return (size_t)(k / 256) * 210;
    case CKQ_FMT_Q8_0: return (size_t)(k / 32) * 34;
    case CKQ_FMT_Q8_K: return (size_t)(k / 256) * 292;
    default: return 0;
    }
}

static void *xmalloc(size_t n)
{
    void *p = malloc(n ? n : 1);
    if (!p) { fprintf(stderr, "out of memory\n"); exit(2); }
    return p;
}

static int all_finite(const float *y, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        if (!isfinite(y[i])) return 0;
    return 1;
}

/* quantizers on edge inputs, matmuls of every format on ragged shapes */
static void run_oracle(void)
{
    static const int ks[] = {256, 512, 1024, 2304};
    for (size_t ki = 0; ki < sizeof ks / sizeof ks[0]; ++ki) {
        const int K = ks[ki], M = 5 + (int)ki, T = 3;
        float *x = xmalloc((size_t)T * K * sizeof(float));
        ckq_synth_normal(x, (size_t)T * K, 0.0f, 1.0f, 11 + ki);
        /* extremes the quantizers special-case: zeros, ties, tiny and huge magnitudes, infinities' neighbours */
        for (int i = 0; i < 32; ++i) x[i] = 0.0f;
        x[40] = 3.0f; x[41] = -3.0f; x[64] = 1e-41f; x[65] = -1e-40f;
        uint8_t *xk = xmalloc((size_t)T * row_bytes(CKQ_FMT_Q8_K, K));
        uint8_t *x0 = xmalloc((size_t)T * row_bytes(CKQ_FMT_Q8_0, K));
        x[96] = 3e38f; x[97] = -3e38f;                      /* the quantizers alone see the huge values */
        orc_quantize_batch_q8_k(x, xk, T, K);
        orc_quantize_batch_q8_0(x, x0, T, K);
        x[96] = 0.5f; x[97] = -0.5f;
        orc_quantize_batch_q8_k(x, xk, T, K);
        orc_quantize_batch_q8_0(x, x0, T, K);
        float *tiny = xmalloc(256 * sizeof(float));
        for (int i = 0; i < 256; ++i) tiny[i] = (i % 3 ? 1.0f : -1.0f) * 1e-39f;   /* infinite inverse scale */
        uint8_t *tk = xmalloc(292), *t0 = xmalloc(8 * 34);
        orc_quantize_row_q8_k(tiny, tk, 256);
        orc_quantize_row_q8_0(tiny, t0, 256);
        CHECK((int8_t)tk[4] == -128);
        float *gam = xmalloc((size_t)K * sizeof(float));
        ckq_synth_normal(gam, K, 1.0f, 0.2f, 5);
        uint8_t *rq = xmalloc((size_t)T * row_bytes(CKQ_FMT_Q8_K, K));
        orc_rmsnorm_q8_k_fused(x, gam, rq, T, K, K, 1e-5f);
        orc_rmsnorm_q8_k_fused_nofma(x, gam, rq, T, K, K, 1e-5f);
        uint8_t *sq = xmalloc((size_t)T * row_bytes(CKQ_FMT_Q8_K, K));
        orc_swiglu_q8_k(x, x, sq, T, K, K);

        static const int fmts[] = {CKQ_FMT_Q4_K, CKQ_FMT_Q5_K, CKQ_FMT_Q6_K, CKQ_FMT_Q8_0};
        for (size_t fi = 0; fi < 4; ++fi) {
            const int fmt = fmts[fi];
            const size_t rb = row_bytes(fmt, K);
            uint8_t *W = xmalloc((size_t)M * rb), *R = xmalloc((size_t)M * rb);
            CHECK(ckq_synth_weights(fmt, W, M, K, 0.0f, 0.02f, 100 + fi) == 0);
            CHECK(ckq_synth_random_blocks(fmt, R, (size_t)M * (fmt == CKQ_FMT_Q8_0 ? K / 32 : K / 256), 200 + fi) == 0);
            const void *act = fmt == CKQ_FMT_Q8_0 ? (const void *)x0 : (const void *)xk;
            float *y = xmalloc((size_t)T * M * sizeof(float)), *bias = xmalloc((size_t)M * sizeof(float));
            double *yd = xmalloc((size_t)M * sizeof(double));
            ckq_synth_normal(bias, M, 0.0f, 0.5f, 7);
            const int nsub = fmt == CKQ_FMT_Q6_K ? K / 16 : K / 32;
            int32_t *sub = xmalloc((size_t)nsub * sizeof(int32_t));
            float *deq = xmalloc((size_t)K * sizeof(float));
            switch (fmt) {
            case CKQ_FMT_Q4_K:
                orc_gemv_q4_k_q8_k(y, W, act, M, K);
                orc_gemm_nt_q4_k_q8_k(act, W, bias, y, T, M, K);
                orc_gemm_q4_k_q8_k(y, R, act, M, T, K);
                orc_gemv_q4_k(y, W, x, M, K);
                orc_gemm_nt_q4_k(x, W, bias, y, T, M, K);
                orc_subdots_q4_k_q8_k(R, act, K, sub);
                orc_dequant_q4_k_row(R, deq, K);
                for (int nth = 1; nth <= 9; nth += 4)
                    for (int ith = 0; ith < nth; ++ith) orc_gemv_q4_k_q8_k_parallel(y, W, act, M, K, ith, nth);
                break;
            case CKQ_FMT_Q5_K:
                orc_gemv_q5_k_q8_k(y, W, act, M, K);
                orc_gemm_nt_q5_k_q8_k(act, W, bias, y, T, M, K);
                orc_gemv_q5_k(y, W, x, M, K);
                orc_gemm_nt_q5_k(x, W, NULL, y, T, M, K);
                orc_subdots_q5_k_q8_k(R, act, K, sub);
                orc_dequant_q5_k_row(R, deq, K);
                break;
            case CKQ_FMT_Q6_K:
                orc_gemv_q6_k_q8_k(y, W, act, M, K);
                orc_gemv_q6_k_q8_k_ref(y, R, act, M, K);
                orc_gemm_nt_q6_k_q8_k(act, W, bias, y, T, M, K);
                orc_gemm_q6_k_q8_k(y, W, act, M, T, K);
                orc_gemv_q6_k(y, W, x, M, K);
                orc_gemm_nt_q6_k(x, W, bias, y, T, M, K);
                orc_vec_dot_q6_k_q8_k(K, y, W, act);
                orc_subdots_q6_k_q8_k(R, act, K, sub);
                orc_dequant_q6_k_row(R, deq, K);
                for (int ith = 0; ith < 7; ++ith) orc_gemv_q6_k_q8_k_parallel(y, W, act, M, K, ith, 7);
                break;
            default:
                orc_gemv_q8_0_q8_0(y, W, act, M, K);
                orc_gemv_q8_0_q8_0_lanes8(y, R, act, M, K);
                orc_gemm_nt_q8_0_q8_0(act, W, bias, y, T, M, K);
                orc_gemv_q8_0(y, W, x, M, K);
                orc_gemm_nt_q8_0(x, W, bias, y, T, M, K);
                orc_vec_dot_q8_0_q8_0(K, y, W, act);
                orc_subdots_q8_0_q8_0(R, act, K, sub);
                orc_dequant_q8_0_row(R, deq, K);
                for (int ith = 0; ith < 3; ++ith) orc_gemv_q8_0_q8_0_parallel(y, W, act, M, K, ith, 3);
                break;
            }
            orc_gemv_exact_f64(fmt, yd, W, act, M, K);
            orc_gemv_threads(fmt, y, W, act, M, K, 3);
            CHECK(all_finite(y, M));
            free(W); free(R); free(y); free(bias); free(yd); free(sub); free(deq);
        }
        /* Q5_0: rewrite to Q8_0 keeps every dot product */
        {
            const size_t nblk = (size_t)M * (K / 32);
            uint8_t *w50 = xmalloc(nblk * 22), *w80 = xmalloc(nblk * 34);
            CHECK(ckq_synth_random_blocks(CKQ_FMT_Q5_0, w50, nblk, 31) == 0);
            orc_q5_0_to_q8_0(w50, w80, nblk);
            float *ya = xmalloc((size_t)M * sizeof(float)), *yb = xmalloc((size_t)M * sizeof(float));
            orc_gemv_q5_0_q8_0(ya, w50, x0, M, K);
            orc_gemv_q8_0_q8_0(yb, w80, x0, M, K);
            orc_gemm_nt_q5_0_q8_0(x0, w50, NULL, ya, 1, M, K);
            free(w50); free(w80); free(ya); free(yb);
        }
        /* embedding lookup with ids outside the vocabulary and a padded row */
        {
            const int vocab = 9, ed = K - 8, ctx = 6;
            uint8_t *tab = xmalloc((size_t)vocab * row_bytes(CKQ_FMT_Q4_K, K));
            CHECK(ckq_synth_weights(CKQ_FMT_Q4_K, tab, vocab, K, 0.0f, 0.02f, 41) == 0);
            const int32_t ids[4] = {3, -1, 8, 9};
            float *pos = xmalloc((size_t)ctx * K * sizeof(float)), *out = xmalloc((size_t)ctx * K * sizeof(float));
            ckq_synth_normal(pos, (size_t)ctx * K, 0.0f, 0.1f, 42);
            orc_embedding_forward(CKQ_FMT_Q4_K, ids, 4, vocab, tab, pos, out, ed, K, ctx, 1);
            CHECK(out[(size_t)5 * K] == 0.0f);
            free(tab); free(pos); free(out);
        }
        free(x); free(xk); free(x0); free(tiny); free(tk); free(t0); free(gam); free(rq); free(sq);
    }
    /* fused prefill MLP: a full tile of 64 tokens and a ragged one */
    {
        const int seq = 70, E = 256, I = 512;
        float *x = xmalloc((size_t)seq * E * sizeof(float)), *out = xmalloc((size_t)seq * E * sizeof(float));
        ckq_synth_normal(x, (size_t)seq * E, 0.0f, 1.0f, 61);
        uint8_t *W1 = xmalloc((size_t)2 * I * row_bytes(CKQ_FMT_Q8_0, E)), *W2 = xmalloc((size_t)E * row_bytes(CKQ_FMT_Q4_K, I));
        CHECK(ckq_synth_weights(CKQ_FMT_Q8_0, W1, 2 * I, E, 0.0f, 0.25f, 62) == 0);
        CHECK(ckq_synth_weights(CKQ_FMT_Q4_K, W2, E, I, 0.0f, 0.02f, 63) == 0);
        float *gu = xmalloc((size_t)seq * 2 * I * sizeof(float));
        uint8_t *hq = xmalloc((size_t)seq * row_bytes(CKQ_FMT_Q8_K, I));
        orc_fused_mlp_swiglu_prefill_w1w2_quant(x, W1, NULL, 9, W2, NULL, 7, out, seq, E, E, I, I, gu, hq);
        CHECK(all_finite(out, (size_t)seq * E));
        free(x); free(out); free(W1); free(W2); free(gu); free(hq);
    }
    /* scalar helpers over their whole domain */
    for (unsigned h = 0; h < 65536; ++h) {
        const float f = orc_fp16_to_fp32((uint16_t)h);
        if (f == f) CHECK(orc_fp32_to_fp16(f) == (uint16_t)h || f == 0.0f);
    }
    for (int v = 0; v < 4096; ++v) {
        uint8_t s12[12], a[8], b[8], c[8], d[8];
        ckq_synth_bytes(s12, 12, 1000 + v);
        orc_unpack_scales_k4(s12, a, b);
        orc_unpack_scales_k4_kmask(s12, c, d);
        CHECK(!memcmp(a, c, 8) && !memcmp(b, d, 8));
    }
}

/* the library's HIP-free host helpers */
static void run_host_helpers(void)
{
    /* row split: the ranges of all threads tile [0, M) in order; whole mode gives everything to thread 0 */
    for (int M = 1; M < 70; ++M)
        for (int nth = 1; nth < 40; ++nth) {
            int next = 0;
            for (int ith = 0; ith < nth; ++ith) {
                int r0 = -1, r1 = -1;
                if (!ckq_split_rows(M, ith, nth, 0, &r0, &r1)) continue;
                CHECK(r0 == next && r1 > r0 && r1 <= M);
                next = r1;
            }
            CHECK(next == M);
            int r0 = -1, r1 = -1;
            CHECK(ckq_split_rows(M, 0, nth, 1, &r0, &r1) && r0 == 0 && r1 == M);
            CHECK(nth == 1 || !ckq_split_rows(M, nth - 1, nth, 1, &r0, &r1));
        }
    {
        int r0, r1;
        CHECK(!ckq_split_rows(10, -1, 4, 0, &r0, &r1) && !ckq_split_rows(10, 4, 4, 0, &r0, &r1) && !ckq_split_rows(10, 0, 0, 0, &r0, &r1));
        CHECK(ckq_split_rows(0x7fffffff, 0x3fffffff, 0x40000000, 0, &r0, &r1));    /* no overflow in the products */
    }
    /* grid chunks */
    static const long cases[][2] = {{1, 65535}, {65535, 65535}, {65536, 65535}, {70000, 65535}, {8 * 65535 + 3, 8 * 65535}};
    for (size_t i = 0; i < sizeof cases / sizeof cases[0]; ++i) {
        long covered = 0, c = 0;
        while (c * cases[i][1] < cases[i][0]) {
            long first, count;
            ckq_grid_chunk(cases[i][0], cases[i][1], c, &first, &count);
            CHECK(first == covered && count > 0 && count <= cases[i][1]);
            covered += count;
            ++c;
        }
        CHECK(covered == cases[i][0]);
    }
    /* fingerprint: every size from empty to beyond the sampled span, exact-size buffers */
    for (size_t n = 0; n < 9000; n += (n < 300 ? 1 : 97)) {
        uint8_t *b = xmalloc(n);
        ckq_synth_bytes(b, n, n);
        const uint64_t h = ckq_fingerprint(b, n);
        if (n) { b[n - 1] ^= 1; if (n <= 64 * 64) CHECK(ckq_fingerprint(b, n) != h); }
        free(b);
    }
    /* overlap predicate at the ends of the address space */
    CHECK(ckq_ranges_overlap((void *)100, 10, (void *)109, 1) && !ckq_ranges_overlap((void *)100, 10, (void *)110, 5));
    CHECK(!ckq_ranges_overlap((void *)100, 0, (void *)100, 0));
    /* workspace slots */
    {
        uint64_t keys[4] = {0}, use[4] = {0};
        for (uint64_t k = 1; k <= 10; ++k) {
            const int i = ckq_workspace_pick(keys, use, 4, (1ull << 63) | k);
            CHECK(i >= 0 && i < 4);
            keys[i] = (1ull << 63) | k;
            use[i] = k;
            CHECK(ckq_workspace_pick(keys, use, 4, keys[i]) == i);
        }
    }
    /* manifest lines: good, skipped and malformed ones, each in a buffer of its exact length */
    static const struct { const char *line; int want; unsigned long long size, off; } lines[] = {
        {"blk.0.attn_q.weight|q4_k|4096|9437184|0x1000\n", 1, 9437184ull, 0x1000ull},
        {"  tok|Q6K|0|210|64", 1, 210ull, 64ull},
        {"w|q8_0|0|0|64\n", 0, 0, 0},                       /* empty tensor */
        {"norm|fp32|0|16384|0\n", 0, 0, 0},
        {"# comment|q4_k|1|2|3\n", 0, 0, 0},
        {"\n", 0, 0, 0}, {"", 0, 0, 0}, {"   \t", 0, 0, 0},
        {"name|q4_k|12|34\n", -1, 0, 0}, {"|", -1, 0, 0}, {"a|b|c|d", -1, 0, 0},
        {"x|q5_0|0|077|010|trailing|fields\n", 1, 63ull, 8ull},
    };
    for (size_t i = 0; i < sizeof lines / sizeof lines[0]; ++i) {
        const size_t n = strlen(lines[i].line) + 1;
        char *buf = xmalloc(n);
        memcpy(buf, lines[i].line, n);
        unsigned long long size = 0, off = 0;
        const int got = ckq_manifest_parse_line(buf, &size, &off);
        CHECK(got == lines[i].want);
        if (got == 1) CHECK(size == lines[i].size && off == lines[i].off);
        free(buf);
    }
}

int main(void)
{
    run_host_helpers();
    run_oracle();
    if (failures) { fprintf(stderr, "asan_harness: %d check(s) failed\n", failures); return 1; }
    printf("asan_harness: ok\n");
    return 0;
}
