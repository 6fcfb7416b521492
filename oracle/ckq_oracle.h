/*
 * ckq_oracle.h - CPU oracle for the quantized dequant-dot matmul path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the reference
 * engine's CPU arithmetic for the Q4_K/Q5_K/Q6_K/Q8_0 x Q8_K/Q8_0 kernels and
 * the fp32->Q8_K / fp32->Q8_0 activation quantizers.  Only the test-suite,
 * the smoke check and the CPU-baseline leg of the benchmark may link or load
 * it; the GPU library never does.
 *
 * Every function names the reference file:line it follows (paths relative to
 * the reference checkout).
 */
#ifndef CKQ_ORACLE_H
#define CKQ_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- scalar helpers ---------------------------------------------------- */
float    orc_fp16_to_fp32(uint16_t h);          /* include/ckernel_quant.h:265-294 */
uint16_t orc_fp32_to_fp16(float f);             /* include/ckernel_quant.h:311-336,355-357 (RNE) */
void     orc_unpack_scales_k4(const uint8_t *s12, uint8_t *sc8, uint8_t *m8);      /* ckernel_quant.h:227-251 */
void     orc_unpack_scales_k4_kmask(const uint8_t *s12, uint8_t *sc8, uint8_t *m8); /* gemm_kernels_q5_k.c:163-170 */

/* ---- activation quantizers (bit-exact contract) ------------------------ */
void orc_quantize_row_q8_k(const float *x, void *y, int k);                 /* quantize_row_q8_k_sse.c:22-82 */
void orc_quantize_batch_q8_k(const float *x, void *y, int rows, int k);     /* gemm_kernels_q8_0.c:221-239 */
void orc_quantize_row_q8_0(const float *x, void *y, int k);                 /* gemm_kernels_q8_0.c:70-146 */
void orc_quantize_batch_q8_0(const float *x, void *y, int rows, int k);     /* gemm_kernels_q8_0.c:194-209 */
/* fused/rmsnorm_q8_k_fused.c:54-142 (as built with FMA; _nofma: product rounded before the add) */
void orc_rmsnorm_q8_k_fused(const float *input, const float *gamma, void *vy, int tokens, int d_model, int aligned_embed_dim, float eps);
void orc_rmsnorm_q8_k_fused_nofma(const float *input, const float *gamma, void *vy, int tokens, int d_model, int aligned_embed_dim, float eps);

/* ---- dequantizers (fp32 cross-check reference) ------------------------- */
void orc_dequant_q4_k_row(const void *src, float *dst, size_t n);           /* dequant_kernels.c:336-385 */
void orc_dequant_q5_k_row(const void *src, float *dst, size_t n);           /* gemm_kernels_q5_k.c:130-208 (layout) */
void orc_dequant_q6_k_row(const void *src, float *dst, size_t n);           /* dequant_kernels.c:396-430 */
void orc_dequant_q8_0_row(const void *src, float *dst, size_t n);           /* dequant_kernels.c:276-296 */
void orc_dequant_q8_k_row(const void *src, float *dst, size_t n);           /* d * qs; block layout ckernel_quant.h:153-157 */
/* src/kernels/embedding_kernels.c:76-260 (fmt: CKQ_FMT_Q4_K, _Q6_K or _Q8_0) */
void orc_embedding_forward(int fmt, const int32_t *token_ids, int token_count, int vocab_size,
                           const void *token_embeddings, const float *pos_embeddings, float *output,
                           int embed_dim, int aligned_embed_dim, int context_window, int add_pos);

/* ---- integer sub-block dots (bit-exact contract) ----------------------- *
 * One weight row against one activation vector.  Output counts per
 * super-block: Q4_K/Q5_K 8 (sum over 32 of q*q8), Q6_K 16 (sum over 16 of
 * (q-32)*q8), Q8_0 1 per 32-block.                                         */
void orc_subdots_q4_k_q8_k(const void *w_row, const void *x_q8, int K, int32_t *out);
void orc_subdots_q5_k_q8_k(const void *w_row, const void *x_q8, int K, int32_t *out);
void orc_subdots_q6_k_q8_k(const void *w_row, const void *x_q8, int K, int32_t *out);
void orc_subdots_q8_0_q8_0(const void *w_row, const void *x_q8, int K, int32_t *out);

/* ---- GEMV: y[M] = W[M x K] . x ----------------------------------------- */
void orc_gemv_q4_k_q8_k(float *y, const void *W, const void *x_q8, int M, int K);      /* gemm_kernels_q4k_q8k.c:121-200 */
/* CPU-baseline timing: persistent threads, one barrier-bracketed round per call of a split GEMV. */
typedef void (*orc_split_gemv_fn)(float *y, const void *W, const void *x_q8, int M, int K, int ith, int nth);
int orc_time_split_gemv(orc_split_gemv_fn fn, float *y, const void *W, const void *x_q8, int M, int K, int nth, int iters,
                        double *seconds);
/* ... over w_copies copies of the weights, w_stride bytes apart, one per round in turn (DRAM-resident weights). */
int orc_time_split_gemv_rotating(orc_split_gemv_fn fn, float *y, const void *W, size_t w_stride, int w_copies,
                                 const void *x_q8, int M, int K, int nth, int iters, double *seconds);
void orc_gemv_q4_k_q8_k_parallel(float *y, const void *W, const void *x_q8, int M, int K, int ith, int nth); /* :212-243 */
void orc_gemv_q5_k_q8_k(float *y, const void *W, const void *x_q8, int M, int K);      /* gemm_kernels_q5_k.c:130-208,305-329 */
void orc_gemv_q5_k(float *y, const void *W, const float *x, int M, int K);             /* gemm_kernels_q5_k.c:369-391 (K%256==0 branch) */
void orc_gemv_q6_k_q8_k_ref(float *y, const void *W, const void *x_q8, int M, int K);  /* gemm_kernels_q6k_q8k.c:70-120,197-214 */
void orc_gemv_q6_k_q8_k(float *y, const void *W, const void *x_q8, int M, int K);      /* gemm_kernels_q6k_q8k.c:601-695 (integer block form, 8 float lanes) */
void orc_gemv_q6_k_q8_k_parallel(float *y, const void *W, const void *x_q8, int M, int K, int ith, int nth); /* :1141-1197 */
void orc_vec_dot_q6_k_q8_k(int n, float *s, const void *vx, const void *vy);           /* gemm_kernels_q6k_q8k.c:1032-1055 */
void orc_gemv_q8_0_q8_0(float *y, const void *W, const void *x_q8, int M, int K);      /* gemm_kernels_q8_0.c:968-989,1237-1251 */
void orc_gemv_q8_0_q8_0_lanes8(float *y, const void *W, const void *x_q8, int M, int K); /* gemm_kernels_q8_0.c:845-889,1031-1058 (AVX2 order) */
void orc_gemv_q8_0_q8_0_parallel(float *y, const void *W, const void *x_q8, int M, int K, int ith, int nth); /* :1263-1287 */
void orc_vec_dot_q8_0_q8_0(int n, float *s, const void *vx, const void *vy);           /* gemm_kernels_q8_0.c:968-989 */
void orc_gemv_q8_0(float *y, const void *W, const float *x, int M, int K);             /* gemm_kernels_q8_0.c:254-277 */
void orc_gemv_q4_k(float *y, const void *W, const float *x, int M, int K);             /* gemm_kernels_q4k.c:53-101 (fp32 activations) */
void orc_gemv_q6_k(float *y, const void *W, const float *x, int M, int K);             /* gemm_kernels_q6k.c:39-76,169-193 (fp32 activations) */

/* ---- GEMM ---------------------------------------------------------------
 * gemm_*   : Y[n*M + row], M = output rows, N = tokens.
 * gemm_nt_*: C[m*N + n],   M = tokens,      N = output rows, optional bias[N]. */
void orc_gemm_q4_k_q8_k(float *Y, const void *W, const void *X_q8, int M, int N, int K);                        /* gemm_kernels_q4k_q8k.c:283-299 */
void orc_gemm_nt_q4_k_q8_k(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K);  /* :301-326 */
void orc_gemm_nt_q5_k_q8_k(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K);  /* gemm_kernels_q5_k.c:331-359 */
void orc_gemm_nt_q5_k(const float *A, const void *B, const float *bias, float *C, int M, int N, int K);         /* gemm_kernels_q5_k.c:401-430 */
void orc_gemm_q6_k_q8_k(float *Y, const void *W, const void *X_q8, int M, int N, int K);                        /* gemm_kernels_q6k_q8k.c:1209-1225 */
void orc_gemm_nt_q6_k_q8_k(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K);  /* :1243-1268 */
void orc_gemm_nt_q8_0_q8_0(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K);  /* gemm_batch_int8.c:87-120,582-610 */
void orc_gemm_q4_k(float *Y, const void *W, const float *X, int M, int N, int K);                                   /* gemm_kernels_q4k.c:316-330,461-469 */
void orc_gemm_nt_q4_k(const float *A, const void *B, const float *bias, float *C, int M, int N, int K);            /* gemm_kernels_q4k.c:683-711 */
void orc_gemm_q6_k(float *Y, const void *W, const float *X, int M, int N, int K);                                   /* gemm_kernels_q6k.c:195-210 */
void orc_gemm_nt_q6_k(const float *A, const void *B, const float *bias, float *C, int M, int N, int K);            /* gemm_kernels_q6k.c:212-240 */
void orc_gemm_nt_q8_0(const float *A, const void *B, const float *bias, float *C, int M, int N, int K);            /* gemm_kernels_q8_0.c:683-696 */

/* ---- Q5_0 weights x Q8_0 activations ---------------------------------------
 * per 32-block: sumi = sum (q5 - 16) * q8, sumf += (fp16(dw) * fp16(dx)) * sumi
 * (gemm_kernels_q5_0.c:901-939; the SIMD dispatches sum the same terms in
 * other orders).                                                            */
void orc_subdots_q5_0_q8_0(const void *w_row, const void *x_q8, int K, int32_t *out);
void orc_vec_dot_q5_0_q8_0(int n, float *s, const void *vx, const void *vy);                                       /* gemm_kernels_q5_0.c:1602-1620 */
void orc_gemv_q5_0_q8_0(float *y, const void *W, const void *x_q8, int M, int K);                                  /* :1637-1657 */
void orc_gemm_nt_q5_0_q8_0(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K);     /* :1725-1753 */
/* Q5_0 block -> the Q8_0 block with the same scale and the values q5 - 16:
 * every dot product of the two is identical.                                */
void orc_q5_0_to_q8_0(const void *src, void *dst, size_t nblocks);

/* ---- fused prefill MLP ----------------------------------------------------
 * fused/prefill_fused_gemm.c:964-1060: Q8_0(x) x W1 (gate rows then up rows),
 * SiLU(gate)*up with the C library's expf, Q8_K of that, x W2.  w1_dt / w2_dt
 * are the reference's CKDataType values (W1: Q8_0 = 9 or Q5_0 = 11; W2: Q4_K = 7
 * or Q6_K = 8); other types return without writing.  gate_up_out (seq_len x 2*aligned_intermediate
 * floats: gate, already multiplied, then up) and h_q8k_out receive the
 * intermediates when non-NULL.                                              */
void orc_fused_mlp_swiglu_prefill_w1w2_quant(const float *x, const void *W1, const float *B1, int w1_dt,
                                             const void *W2, const float *B2, int w2_dt, float *output,
                                             int seq_len, int embed_dim, int aligned_embed_dim,
                                             int intermediate_dim, int aligned_intermediate_dim,
                                             float *gate_up_out, void *h_q8k_out);
/* Q8_K of SiLU(gate)*up, rows ld floats apart (fused/prefill_fused_gemm.c:904-906,1034-1047). */
void orc_swiglu_q8_k(const float *gate, const float *up, void *y, int rows, int k, long ld);

/* ---- exact evaluation ---------------------------------------------------
 * Same integers, block scales combined in double: the value every fp32
 * summation order approximates.  fmt is a ckq_format weight tag; the
 * activation format is Q8_0 for CKQ_FMT_Q8_0 weights and Q8_K otherwise.   */
void orc_gemv_exact_f64(int fmt, double *y, const void *W, const void *x_q8, int M, int K);

/* Row-split multi-threaded GEMV used by the CPU-baseline timing: rows
 * [ith*ceil(M/nth), ...) per thread as in gemm_kernels_q4k_q8k.c:226-231.  */
void orc_gemv_threads(int fmt, float *y, const void *W, const void *x_q8, int M, int K, int nth);

#ifdef __cplusplus
}
#endif
#endif
