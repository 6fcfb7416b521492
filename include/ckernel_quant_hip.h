/*
 * ckernel_quant_hip.h - C ABI of libckernel_quant_hip.so, the MI355X (gfx950)
 * implementation of the C-Kernel-Engine quantized dequant-dot matmul path.
 *
 * Part 1 re-exports, with identical names, signatures, argument meaning and
 * error behaviour, the reference's kernel symbols for this path, so a
 * generated libmodel.so (or libck_parity.so users) can link against this
 * library instead of the CPU kernels.  Pointers may be HOST pointers (as the
 * reference passes them) or DEVICE pointers; host buffers are staged, weight
 * matrices are uploaded once and kept resident (see ckq_weights_*).
 * Like the reference: void return, NULL pointer or non-positive dimension
 * returns without touching the output.
 *
 * Part 2 (`ckq_*_dev`) is the same arithmetic on device-resident buffers with
 * an explicit stream and an int status; nothing is copied or synchronized.
 *
 * Naming trap kept from the reference: in gemv_* M = output rows, K = input
 * width; in gemm_nt_* M = tokens, N = output rows; in gemm_*_q8_k(Y,W,X,M,N,K)
 * M = output rows, N = tokens and Y[n*M + row].
 */
#ifndef CKERNEL_QUANT_HIP_H
#define CKERNEL_QUANT_HIP_H

#include <stddef.h>
#include <stdint.h>
#include "ckq_blocks.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ======================================================================== */
/* Part 1: drop-in symbols (reference declarations: include/ckernel_engine.h */
/* :192-363 and include/ckernel_quant.h:398-410)                             */
/* ======================================================================== */

/* fp32 -> Q8_K, k % 256 == 0.  Replaces src/kernels/gemm_kernels_q4k_q8k.c:109-119
 * (dispatch) -> quantize_row_q8_k_sse.c:22-82.  Bit-exact. */
void quantize_row_q8_k(const float *x, void *y, int k);
/* Row loop, output stride (k/256)*292.  Replaces gemm_kernels_q8_0.c:221-239. */
void quantize_batch_q8_k(const float *x, void *y, int num_rows, int k);
/* fp32 -> Q8_0, k % 32 == 0.  Replaces gemm_kernels_q8_0.c:70-175.  Bit-exact. */
void quantize_row_q8_0(const float *x, void *y, int k);
/* Replaces gemm_kernels_q8_0.c:194-209. */
void quantize_batch_q8_0(const float *x, void *y, int num_rows, int k);

/* Q4_K x Q8_K.  Replace gemm_kernels_q4k_q8k.c:245-263 (dispatch), :183-200 (_ref). */
void gemv_q4_k_q8_k(float *y, const void *W, const void *x_q8, int M, int K);
void gemv_q4_k_q8_k_ref(float *y, const void *W, const void *x_q8, int M, int K);
/* Thread-split variants: rows [ith*ceil(M/nth), ...) only.  Replace
 * gemm_kernels_q4k_q8k.c:212-243 and gemm_kernels_q4k_avx.c:136-245. */
void gemv_q4_k_q8_k_parallel(float *y, const void *W, const void *x_q8, int M, int K, int ith, int nth);
void gemv_q4_k_q8_k_parallel_simd(float *y, const void *W, const void *x_q8, int M, int K, int ith, int nth);
/* Y[n*M + row].  Replaces gemm_kernels_q4k_q8k.c:283-299. */
void gemm_q4_k_q8_k(float *Y, const void *W, const void *X_q8, int M, int N, int K);
/* C[m*N + n] (+bias[n]).  Replaces gemm_kernels_q4k_q8k.c:301-326. */
void gemm_nt_q4_k_q8_k(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K);

/* Q5_K.  Replace gemm_kernels_q5_k.c:436-456 (gemv_q5_k_q8_k), :458-479
 * (gemm_nt_q5_k_q8_k), :481-498 (gemv_q5_k) and :500-521 (gemm_nt_q5_k).  The
 * fp32 adapters quantize the activations to Q8_K first; K % 256 != 0 returns
 * without writing (the reference's non-GGUF fp32 fallback is not provided). */
void gemv_q5_k_q8_k(float *y, const void *W, const void *x_q8, int M, int K);
void gemm_nt_q5_k_q8_k(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K);
void gemv_q5_k(float *y, const void *W, const float *x, int M, int K);
void gemm_nt_q5_k(const float *A, const void *B, const float *bias, float *C, int M, int N, int K);

/* Q6_K x Q8_K.  Replace gemm_kernels_q6k_q8k.c:1032-1055 (vec_dot), :1060-1088
 * (gemv), :1105-1197 (_parallel, _parallel_simd), :1209-1225 (gemm), :1243-1268
 * (gemm_nt). */
void vec_dot_q6_k_q8_k(int n, float *s, const void *vx, const void *vy);
void gemv_q6_k_q8_k(float *y, const void *W, const void *x_q8, int M, int K);
void gemv_q6_k_q8_k_parallel(float *y, const void *W, const void *x_q8, int M, int K, int ith, int nth);
void gemv_q6_k_q8_k_parallel_simd(float *y, const void *W, const void *x_q8, int M, int K, int ith, int nth);
void gemm_q6_k_q8_k(float *Y, const void *W, const void *X_q8, int M, int N, int K);
void gemm_nt_q6_k_q8_k(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K);

/* Q8_0.  Replace gemm_kernels_q8_0.c:1204-1219 (vec_dot), :1237-1251 (gemv
 * q8_0 x q8_0), :1263-1343 (_parallel, _parallel_simd), :632-649 (gemv_q8_0,
 * fp32 activations) and gemm_batch_int8.c:582-610 (gemm_nt_q8_0_q8_0). */
void vec_dot_q8_0_q8_0(int n, float *s, const void *vx, const void *vy);
void gemv_q8_0_q8_0(float *y, const void *W, const void *x_q8, int M, int K);
void gemv_q8_0_q8_0_parallel(float *y, const void *W, const void *x_q8, int M, int K, int ith, int nth);
void gemv_q8_0_q8_0_parallel_simd(float *y, const void *W, const void *x_q8, int M, int K, int ith, int nth);
void gemv_q8_0(float *y, const void *W, const float *x, int M, int K);
void gemm_nt_q8_0_q8_0(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K);

/* fp32 activations used as they are: the weights are dequantized on the fly,
 * nothing is quantized.  Same naming trap as above (gemv: M rows; gemm_q*:
 * Y[n*M + row]; gemm_nt: M tokens, N rows).  Replace gemm_kernels_q4k.c:285-297
 * (gemv_q4_k), :461-469 (gemm_q4_k), :484-489 (dot_q4_k), :683-711
 * (gemm_nt_q4_k); gemm_kernels_q6k.c:169-193 (gemv_q6_k), :195-210 (gemm_q6_k),
 * :212-240 (gemm_nt_q6_k); gemm_kernels_q8_0.c:658-666 (gemm_q8_0), :683-696
 * (gemm_nt_q8_0).  K must be a multiple of the block size (the reference reads
 * whole blocks); otherwise nothing is written. */
void  gemv_q4_k(float *y, const void *W, const float *x, int M, int K);
void  gemm_q4_k(float *Y, const void *W, const float *X, int M, int N, int K);
void  gemm_nt_q4_k(const float *A, const void *B, const float *bias, float *C, int M, int N, int K);
float dot_q4_k(const void *w_q4k, const float *x, int K);
void  gemv_q6_k(float *y, const void *W, const float *x, int M, int K);
void  gemm_q6_k(float *Y, const void *W, const float *X, int M, int N, int K);
void  gemm_nt_q6_k(const float *A, const void *B, const float *bias, float *C, int M, int N, int K);
void  gemm_q8_0(float *Y, const void *W, const float *X, int M, int N, int K);
void  gemm_nt_q8_0(const float *A, const void *B, const float *bias, float *C, int M, int N, int K);

/* Row dequantizers and the quantized embedding lookups built on them (the
 * same block decoders, at the model's input); outputs bit-exact with the
 * reference.  n_elements / aligned_embed_dim must be a multiple of the block
 * size.  embedding_forward_*: out[t] = dequant(table[id[t]]) (+ pos[t] when
 * add_pos and pos_embeddings), ids outside [0,vocab) read row 0, elements from
 * embed_dim on and rows from token_count on are zero.  Replace
 * dequant_kernels.c:276-296,336-385,396-430 and
 * src/kernels/embedding_kernels.c:76-260. */
void dequant_q4_k_row(const void *src, float *dst, size_t n_elements);
void dequant_q6_k_row(const void *src, float *dst, size_t n_elements);
void dequant_q8_0_row(const void *src, float *dst, size_t n_elements);
void embedding_forward_q4_k(const int32_t *token_ids, int token_count, int vocab_size, const void *token_embeddings,
                            const float *pos_embeddings, float *output, int embed_dim, int aligned_embed_dim,
                            int context_window, int add_pos);
void embedding_forward_q6_k(const int32_t *token_ids, int token_count, int vocab_size, const void *token_embeddings,
                            const float *pos_embeddings, float *output, int embed_dim, int aligned_embed_dim,
                            int context_window, int add_pos);
void embedding_forward_q8_0(const int32_t *token_ids, int token_count, int vocab_size, const void *token_embeddings,
                            const float *pos_embeddings, float *output, int embed_dim, int aligned_embed_dim,
                            int context_window, int add_pos);

/* Fused producer of the path's activations: RMSNorm over d_model floats per
 * token (row stride aligned_embed_dim floats) times gamma, quantized to Q8_K
 * in the same pass; vy receives tokens x (d_model/256) blocks.  The block scale
 * comes from the largest |value| (unlike quantize_row_q8_k's signed
 * first-largest), so d is negative.  Bit-exact with the reference built with
 * FMA enabled (every AVX2 host build).  d_model must be a multiple of 256.
 * Replaces src/kernels/fused/rmsnorm_q8_k_fused.c:54-142. */
void rmsnorm_q8_k_fused(const float *input, const float *gamma, void *vy, int tokens, int d_model,
                        int aligned_embed_dim, float eps);

/* Q5_0 weights (fp16 d, 32 five-bit values q - 16 per 22-byte block: the
 * format GGUF files use for rows too short for K-quants) against Q8_0
 * activations.  When the launch picks the matrix cores (more than eight tokens
 * and enough weight bytes, see ckq_set_gemm_policy) the blocks are rewritten as
 * Q8_0 blocks on the device (same scale, values q - 16: every dot product is
 * unchanged) and the Q8_0 matrix-core GEMM runs.  Replaces src/kernels/gemm_kernels_q5_0.c:1602-1620
 * (vec_dot), :1637-1657 (gemv), :1659-1700 (_parallel_simd), :1725-1753 (gemm_nt).
 * The fp32-activation forms gemv_q5_0 / gemm_nt_q5_0 are not built. */
void vec_dot_q5_0_q8_0(int n, float *s, const void *vx, const void *vy);
void gemv_q5_0_q8_0(float *y, const void *W, const void *x_q8, int M, int K);
void gemv_q5_0_q8_0_parallel_simd(float *y, const void *W, const void *x_q8, int M, int K, int ith, int nth);
void gemm_nt_q5_0_q8_0(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K);

/* Fused prefill MLP around the quantized GEMMs: x (seq_len rows of
 * aligned_embed_dim floats) is quantized to Q8_0, multiplied with W1 = [gate
 * rows; up rows] (2 * aligned_intermediate_dim rows, bias B1 of the same length
 * or NULL), SiLU(gate) * up is quantized to Q8_K and multiplied with W2
 * (aligned_embed_dim rows, bias B2 or NULL) into output (seq_len rows of
 * aligned_embed_dim floats).  w1_dt / w2_dt are the reference's CKDataType
 * values (include/ckernel_dtype.h:27-50): W1 CKQ_CK_DT_Q8_0 or CKQ_CK_DT_Q5_0, W2
 * CKQ_CK_DT_Q4_K or CKQ_CK_DT_Q6_K, as in the reference; other types and other
 * argument errors return without touching output, as the reference does.  `scratch` must be non-NULL as in
 * the reference but is not used: intermediates stay in device memory.  Any mix
 * of host and device pointers; synchronous.  The SiLU uses an exponential
 * rounded once from double, so the Q8_K intermediate can differ from a glibc
 * host's by one unit in rare quants; the output agrees within the fp32
 * tolerance of the GEMMs.
 * Replaces src/kernels/fused/prefill_fused_gemm.c:964-1060 and :1062-1080. */
#define CKQ_CK_DT_Q4_K 7
#define CKQ_CK_DT_Q6_K 8
#define CKQ_CK_DT_Q8_0 9
#define CKQ_CK_DT_Q5_0 11
/* The dtype parameters have the reference's own enum type when its header
 * (include/ckernel_dtype.h:27-50, guard CKERNEL_DTYPE_H) has been included
 * before this one, so both declarations of the function agree in one
 * translation unit; otherwise an enum of the same enumerator values (and so
 * the same size and calling convention) stands in for it. */
#ifdef CKERNEL_DTYPE_H
typedef CKDataType ckq_ck_dtype;
#else
typedef enum {
    CKQ_CK_DTYPE_FP32 = 0, CKQ_CK_DTYPE_BF16, CKQ_CK_DTYPE_FP16, CKQ_CK_DTYPE_INT8, CKQ_CK_DTYPE_INT4,
    CKQ_CK_DTYPE_Q4_0, CKQ_CK_DTYPE_Q4_1, CKQ_CK_DTYPE_Q4_K, CKQ_CK_DTYPE_Q6_K, CKQ_CK_DTYPE_Q8_0,
    CKQ_CK_DTYPE_Q8_K, CKQ_CK_DTYPE_Q5_0, CKQ_CK_DTYPE_Q5_1, CKQ_CK_DTYPE_Q5_K, CKQ_CK_DTYPE_COUNT
} ckq_ck_dtype;
#endif
void fused_mlp_swiglu_prefill_w1w2_quant(const float *x, const void *W1, const float *B1, ckq_ck_dtype w1_dt,
                                         const void *W2, const float *B2, ckq_ck_dtype w2_dt, float *output,
                                         int seq_len, int embed_dim, int aligned_embed_dim,
                                         int intermediate_dim, int aligned_intermediate_dim, void *scratch);
size_t fused_mlp_swiglu_prefill_w1w2_quant_scratch_size(int aligned_embed_dim, int aligned_intermediate_dim);

/* Parity-test wrappers: fp32 input is quantized, then the kernel runs.
 * Replace src/ck_parity_api.c:189-197 (dequant), :207-210 (quantize), :217-258 (gemv q4_k/q6_k),
 * :288-360 (gemv q8_0), :397-400 (vec_dot), :411-503 (gemm) and the size
 * getters of include/ck_parity_api.h:614-629. */
void ck_test_quantize_q8_k(const float *src, void *dst, int n);
/* include/ck_parity_api.h:48-53, src/ck_parity_api.c:189-197: the row dequantizers under their parity names */
void ck_test_dequant_q4_k(const void *src, float *dst, int n);
void ck_test_dequant_q6_k(const void *src, float *dst, int n);
void ck_test_gemv_q4_k(const void *weight_q4k, const float *input_f32, float *output, int cols);
void ck_test_gemv_q6_k(const void *weight_q6k, const float *input_f32, float *output, int cols);
void ck_test_gemv_q8_0(const void *weight_q8_0, const float *input_f32, float *output, int rows, int cols);
void ck_test_gemv_q8_0_q8_0(const void *weight_q8_0, const float *input_f32, float *output, int rows, int cols);
void ck_test_vec_dot_q8_0_q8_0(const void *weight_q8_0, const void *input_q8_0, float *output, int cols);
void ck_test_gemm_q4_k(const void *weight_q4k, const float *input_f32, float *output, int rows, int cols, int n_tokens);
void ck_test_gemm_q6_k(const void *weight_q6k, const float *input_f32, float *output, int rows, int cols, int n_tokens);
void ck_test_gemm_q8_0(const void *weight_q8_0, const float *input_f32, float *output, int rows, int cols, int n_tokens);
int  ck_get_block_q4_k_size(void);
int  ck_get_block_q6_k_size(void);
int  ck_get_block_q8_k_size(void);
int  ck_get_qk_k(void);

/* ======================================================================== */
/* Part 2: device-resident entry points                                      */
/* ======================================================================== */
/* All pointers are device pointers; `stream` is a hipStream_t (NULL = null
 * stream); work is enqueued, never synchronized.  Outputs must not overlap
 * inputs.  Return 0, or a negative CKQ_E* / positive hipError_t code.
 * Alignment: Q4_K/Q5_K weights and Q8_K activations 4 bytes, Q6_K/Q8_0 2
 * bytes, fp32 inputs of the quantizers 16 bytes, other fp32 4 bytes. */

int ckq_quantize_q8_k_dev(const float *x, void *y, int num_rows, int k, void *stream);
int ckq_quantize_q8_0_dev(const float *x, void *y, int num_rows, int k, void *stream);

/* Generic form: fmt is a ckq_format weight tag (activations Q8_0 for
 * CKQ_FMT_Q8_0, Q8_K otherwise).  C[m*ldc + n] = dot(B[n], A[m]) (+bias[n]),
 * m < M tokens, n < N rows.  M = 1 with ldc = N is the GEMV. */
int ckq_gemm_nt_dev(int fmt, const void *A_q8, const void *B, const float *bias, float *C,
                    int M, int N, int K, long ldc, void *stream);

/* ckq_gemm_nt_dev for callers that cannot allocate device memory.  It has no
 * counterpart in the reference; it is for code under HIP graph capture, tight
 * serving loops and harnesses that forbid hipMalloc.  Same arithmetic, same
 * kernel choice and the same bits as ckq_gemm_nt_dev (formats CKQ_FMT_Q4_K,
 * _Q5_K, _Q6_K, _Q8_0); the partial tiles of a K-split matrix-core GEMM live in
 * a static device array of 4 MiB (one copy per GPU, held until the process
 * ends) instead of the library's grow-only workspace.  A call whose split
 * needs more (splits x M x N x 4 bytes; up to 16 splits are taken when the
 * tile grid is smaller than the chip) returns CKQ_ESCRATCH (-4) and enqueues
 * nothing: pass fewer tokens per call, or use ckq_gemm_nt_dev; no call allocates,
 * frees or synchronizes.  Every call on a GPU shares that GPU's array: calls
 * that overlap on one GPU (two streams, two threads) race.  The array's
 * address is resolved once per device, by ckq_init() or by the first call on
 * that device; resolving it may load the library's code object, so call
 * ckq_init() on the device BEFORE a region that must not allocate, and before
 * stream capture begins: a first call on a capturing stream with the address
 * still unresolved returns hipErrorStreamCaptureUnsupported. */
int ckq_gemm_nt_noalloc_dev(int fmt, const void *A_q8, const void *B, const float *bias, float *C,
                            int M, int N, int K, long ldc, void *stream);

/* Named forms mirroring Part 1. */
int ckq_gemv_q4_k_q8_k_dev(float *y, const void *W, const void *x_q8, int M, int K, void *stream);
int ckq_gemv_q5_k_q8_k_dev(float *y, const void *W, const void *x_q8, int M, int K, void *stream);
int ckq_gemv_q6_k_q8_k_dev(float *y, const void *W, const void *x_q8, int M, int K, void *stream);
int ckq_gemv_q8_0_q8_0_dev(float *y, const void *W, const void *x_q8, int M, int K, void *stream);
int ckq_gemv_q8_0_dev(float *y, const void *W, const float *x, int M, int K, void *stream);
int ckq_gemm_nt_q4_k_q8_k_dev(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K, void *stream);
int ckq_gemm_nt_q5_k_q8_k_dev(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K, void *stream);
int ckq_gemm_nt_q6_k_q8_k_dev(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K, void *stream);
int ckq_gemm_nt_q8_0_q8_0_dev(const void *A_q8, const void *B, const float *bias, float *C, int M, int N, int K, void *stream);

/* Device form of the dequantizers / embedding lookups: out[t] (n_row floats,
 * 16-byte aligned, t < n_out_rows) = row (ids ? ids[t] clamped : t) of `table`
 * for t < tokens, plus pos[t] when pos is non-NULL, zero from element n_valid
 * on; rows from `tokens` on are zero.  fmt: CKQ_FMT_Q4_K, _Q6_K or _Q8_0. */
int ckq_dequant_rows_dev(int fmt, const void *table, const int32_t *ids, int vocab, const float *pos, float *out,
                         int n_valid, int n_row, int tokens, int n_out_rows, void *stream);

/* Device form of rmsnorm_q8_k_fused; input rows and gamma 16-byte aligned,
 * d_model <= 40 000 (the row is staged in LDS). */
int ckq_rmsnorm_q8_k_fused_dev(const float *input, const float *gamma, void *y, int tokens, int d_model,
                               int aligned_embed_dim, float eps, void *stream);

/* y[row] = Q8_K(SiLU(gate[row]) * up[row]): the step between the two GEMMs of
 * the fused prefill MLP.  k floats per row (multiple of 256), rows of gate and
 * of up ld floats apart, both 16-byte aligned. */
int ckq_swiglu_q8_k_dev(const float *gate, const float *up, void *y, int rows, int k, long ld, void *stream);

/* fp32 activations (M rows of K floats, 16-byte aligned) against `fmt` weights
 * (CKQ_FMT_Q4_K, _Q6_K or _Q8_0), no activation quantization: the device form
 * of gemv_q4_k / gemm_nt_q4_k / gemm_nt_q6_k / gemm_nt_q8_0 above. */
int ckq_gemm_nt_f32act_dev(int fmt, const float *A, const void *B, const float *bias, float *C,
                           int M, int N, int K, long ldc, void *stream);

/* A list of steps enqueued back-to-back, the whole list `repeat` times: the
 * per-token chain of a decoder layer (norm -> Q8_K -> Q/K/V ... -> down) is one
 * such list.  A matmul entry (fmt = a ckq_format weight tag) computes
 * C[m*ldc + n] as ckq_gemm_nt_dev does, with the same bits.  Up to four
 * consecutive matmul entries of one format, input width and token count (their
 * row counts may differ), none of which writes memory another reads or writes
 * (Q/K/V, gate/up), are issued as ONE launch: up to eight tokens by the
 * weight-streaming kernel; beyond that, when the entries also read the same
 * activations and their tiles together fill the chip, by the matrix-core GEMM
 * (a prefill's K and V projections then share the grid of Q instead of taking a
 * K-split launch each; every tile is computed as the unsplit single launch
 * computes it, so an entry whose single launch would be split along K gets the
 * unsplit summation order).  ckq_set_prefill_grouping(0) issues entries of more
 * than eight tokens one by one.  A producer entry (fmt = one of CKQ_STEP_*) runs the activation
 * quantizer that feeds the matmuls after it, so that a whole chain is one C
 * call:
 *   CKQ_STEP_QUANTIZE_Q8_K  C = Q8_K blocks of the M rows of K floats at A_q8 (contiguous rows)
 *   CKQ_STEP_QUANTIZE_Q8_0  the same with Q8_0 blocks
 *   CKQ_STEP_RMSNORM_Q8_K   C = Q8_K(RMSNorm(row) * gamma): M rows of K floats at A_q8, rows ldc floats
 *                           apart (0 = K), gamma at B, epsilon in eps (rmsnorm_q8_k_fused)
 *   CKQ_STEP_SWIGLU_Q8_K    C = Q8_K(SiLU(gate) * up): gate at A_q8, up at B, M rows of K floats, rows
 *                           ldc floats apart (0 = K) (ckq_swiglu_q8_k_dev)
 * N and bias are unused by producer entries; C is the block buffer. */
/* Added to a matmul entry's weight tag (CKQ_FMT_Q4_K, _Q6_K or _Q8_0): the
 * activations at A_q8 are M rows of K floats and the entry computes what
 * ckq_gemm_nt_f32act_dev computes (no activation quantization). */
#define CKQ_ACT_F32 0x200
#define CKQ_STEP_QUANTIZE_Q8_K 32
#define CKQ_STEP_QUANTIZE_Q8_0 33
#define CKQ_STEP_RMSNORM_Q8_K  34
#define CKQ_STEP_SWIGLU_Q8_K   35
typedef struct {
    int          fmt;    /* ckq_format weight tag, or a CKQ_STEP_* producer tag */
    int          M;      /* tokens */
    int          N;      /* output rows */
    int          K;      /* input width */
    long         ldc;    /* output row stride (elements); producers: input row stride */
    const void  *A_q8;   /* activations, M rows; producers: fp32 input */
    const void  *B;      /* weights, N rows; producers: gamma / up */
    const float *bias;   /* N, or NULL */
    float       *C;      /* M x ldc; producers: the quantized blocks */
    float        eps;    /* CKQ_STEP_RMSNORM_Q8_K only */
} ckq_matmul_op;
int ckq_matmul_sequence_dev(const ckq_matmul_op *ops, int nops, int repeat, void *stream);

/* Raw integer sub-block dots of W (M rows) against one activation row, as the
 * GEMV kernel computes them: out[row*(K/sub) + i], sub = 32 (Q4_K, Q5_K, Q8_0)
 * or 16 (Q6_K, sum of (q-32)*q8).  For the bit-exactness tests. */
int ckq_subblock_dots_dev(int fmt, int32_t *out, const void *W, const void *x_q8, int M, int K, void *stream);

/* The same dump for up to eight tokens, taken from the instantiation of the
 * streaming kernel that ckq_gemm_nt_dev would run for this shape and token
 * count (token tile, rows per wave, block size, staged activations):
 * out[(t * M + row) * (K/sub) + i]. */
int ckq_subblock_dots_tokens_dev(int fmt, int32_t *out, const void *W, const void *X_q8, int M, int K, int ntok, void *stream);
/* And from the grouped launch of n (2..4) matmuls of one format, input width
 * and token count that ckq_matmul_sequence_dev issues for independent entries:
 * out[((g * ntok + t) * max_rows + row) * (K/sub) + i], max_rows = the largest
 * rows[g]; W, X_q8 and rows are host arrays of n entries.  Returns CKQ_EINVAL
 * when such a group would be issued as separate launches. */
int ckq_subblock_dots_group_dev(int fmt, int n, int32_t *out, const void *const *W, const void *const *X_q8, const int *rows,
                                int K, int ntok, void *stream);
/* The matrix-core GEMM of `fmt` (whatever the token count and the policy) with
 * the exact integer sums behind every output stored next to the result C[M,N]:
 * sums[((t * N + n) * nblk + b) * per + i]; Q4_K and Q5_K: nblk = K/256, per = 2
 * (I1 = sum sc * sub-block dot, I2 = sum min * stored bsum pair); Q6_K: nblk =
 * K/256, per = 1 (sum sc * 16-run dot of q - 32); Q8_0: nblk = K/32, per = 1
 * (the block dot).  For the bit-exactness tests of the prefill path. */
int ckq_gemm_block_sums_dev(int fmt, const void *A_q8, const void *B, const float *bias, float *C, int32_t *sums,
                            int M, int N, int K, void *stream);

/* Streaming device copy of `bytes` (multiple of 16): calibration kernel for
 * memory counters. */
int ckq_copy_dev(void *dst, const void *src, size_t bytes, void *stream);

/* Streaming device read of the first `bytes & ~15` bytes of src, results
 * discarded (`sink`: 4 writable device bytes that stay untouched).  One launch
 * of it is the time floor of a GEMV whose weights are `bytes` large; the
 * benchmark reports it beside the GEMV figure. */
int ckq_read_dev(const void *src, size_t bytes, void *sink, void *stream);
/* The same read as a tuned streaming kernel: `blocks` blocks of 256 threads
 * stride through the buffer, every lane with `unroll` (1, 2, 4 or 8)
 * independent 16-byte loads in flight per trip.  The benchmark searches
 * (blocks, unroll) and reports the fastest as the launch floor. */
int ckq_read_tuned_dev(const void *src, size_t bytes, void *sink, int blocks, int unroll, void *stream);

/* ======================================================================== */
/* Library control                                                           */
/* ======================================================================== */
/* Explicit initialisation (optional; every entry point initialises lazily).
 * Returns 0 or a hipError_t; fails when no gfx950 device is usable. */
int ckq_init(void);
/* Wait for all work the host-pointer entry points enqueued. */
int ckq_synchronize(void);
/* Weight residency: host weight matrices are uploaded on first use and cached
 * by (address, bytes, fingerprint).  invalidate = drop the region starting at W;
 * clear = drop all; set_cache(0) = upload on every call.
 * register = upload now and pin: a registered region serves every later call
 * whose weights lie anywhere inside it (a whole weight arena can be registered
 * once) and its content is not re-checked until it is invalidated.
 * register_manifest is the loader hook: it reads the weights manifest the
 * reference's loader reads (one tensor per line,
 * name|dtype|file_offset|size|runtime_offset; version/v7/src/
 * ckernel_model_load_v7.c:17-35, 330-377) and registers every q4_k / q5_k /
 * q6_k / q8_0 / q5_0 tensor (names compared without case, with or without the
 * underscore) at base + runtime_offset, base being the arena
 * ck_load_weights filled.  Returns the number of tensors registered or a
 * negative CKQ_E* code (unreadable file, malformed line).
 * resident = number of resident regions, total size through *bytes. */
int  ckq_weights_register(const void *W, size_t bytes);
int  ckq_weights_register_manifest(const void *base, const char *manifest_path);
int  ckq_weights_resident(size_t *bytes);
void ckq_weights_invalidate(const void *W);
void ckq_weights_clear(void);
void ckq_weights_set_cache(int enabled);
/* Bound on the bytes of resident weights that are not registered (0 = the
 * default of 64 GiB; CKQ_WEIGHT_CACHE_MB sets it from the environment).  The
 * least recently used entries are dropped first, never one the running call
 * uses; an operand that does not fit beside those is uploaded for the call
 * and not kept. */
void ckq_weights_set_limit(size_t bytes);
/* Frees the device scratch the library keeps for `stream` (a hipStream_t) on
 * the current device: the partial tiles of K-split GEMMs and rewritten Q5_0
 * weights.  Call it before destroying a stream that ran ckq_*_dev calls. */
int  ckq_release_stream(void *stream);
/* 1 (the default): ckq_matmul_sequence_dev issues independent consecutive entries of
 * more than eight tokens that share their activations as one matrix-core launch;
 * 0: one launch per entry.  No counterpart in the reference. */
void ckq_set_prefill_grouping(int enabled);
/* Thread-split entry points (*_parallel, *_parallel_simd): 0 (the default;
 * CKQ_PARALLEL_MODE=rows) = every call computes exactly the row range of its
 * ith, as the reference does (gemm_kernels_q4k_q8k.c:212-231), so a caller
 * that invokes single ith values or reads its rows before a barrier is served;
 * 1 (CKQ_PARALLEL_MODE=whole) = the ith == 0 call computes all rows in one
 * launch and the other threads return at once - for a thread pool that calls
 * every ith and joins at a barrier, like the reference's (one upload, launch
 * and download instead of nth serialized ones: 5 to 9 times faster per
 * dispatch); a negative value restores the default. */
void ckq_set_parallel_whole(int enabled);
/* Which kernel serves a matmul of more than eight tokens (up to eight always
 * take the weight-streaming kernel, one pass over the weights).  AUTO, the
 * default, picks by token count and weight size: the streaming kernel while
 * its passes over the weights are cheaper than the matrix-core GEMM's fixed
 * cost, the matrix cores beyond.  MATRIX and STREAM force one of them (tests,
 * tuning); CKQ_GEMM_POLICY=matrix|stream sets it from the environment.  Both
 * kernels meet the same tolerance; their fp32 summation orders differ. */
enum { CKQ_GEMM_AUTO = 0, CKQ_GEMM_MATRIX = 1, CKQ_GEMM_STREAM = 2 };
void ckq_set_gemm_policy(int policy);
/* Variants of the matrix-core GEMMs (tests, tuning; 0, the default, picks by shape).  Every variant of a format computes
 * the same sums in the same order: results are bit-identical wherever neither launch splits K or puts two wave groups
 * on a tile.
 *   CKQ_FMT_Q4_K: 64 or 96 = tiles of 128 rows x 64 tokens, or x 96 tokens - fewer instructions per token in blocks that run
 *                 longer, taken where they fit one round that 64-token tiles would not, or the grid is a round and a half deep
 *                 (CKQ_Q4K_TILE=64|96 in the environment);
 *   CKQ_FMT_Q6_K: 1 = one block per CU (64-token tiles three LDS stages deep, 128-token tiles two), 2 = two blocks per CU
 *                 on 64-token tiles with one LDS image of the weights, taken where the 128-token grid would waste a
 *                 quarter or more of its last round (CKQ_Q6K_VARIANT=1|2);
 *   CKQ_FMT_Q5_K: 1 = one block per CU, three LDS stages deep, 2 = two blocks per CU with one LDS image of the weights,
 *                 taken for more tiles than CUs (CKQ_Q5K_VARIANT=1|2).
 * Q8_0 has one variant. */
void ckq_set_prefill_variant(int fmt, int variant);
/* Last error of the calling process (0 = none), its text, and a reset for
 * callers that run with CKQ_ABORT_ON_ERROR=0 and handle errors themselves. */
int         ckq_last_error(void);
void        ckq_clear_error(void);
const char *ckq_error_string(int code);

#ifdef __cplusplus
}
#endif
#endif /* CKERNEL_QUANT_HIP_H */
