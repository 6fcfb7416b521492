/*
 * ckq_launch.h - C interface between the host layer (plain C) and the HIP
 * translation unit.  Every function takes DEVICE pointers and enqueues work on
 * `stream` (a hipStream_t passed as void*; NULL = the null stream); none of
 * them synchronizes.  Return value: 0 on success, a negative CKQ_E* code for a
 * rejected argument, or a positive hipError_t.
 */
#ifndef CKQ_LAUNCH_H
#define CKQ_LAUNCH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CKQ_EINVAL  (-1)  /* NULL pointer / non-positive dimension */
#define CKQ_ESHAPE  (-2)  /* K not a multiple of the block size */
#define CKQ_EFORMAT (-3)  /* unknown format tag */
#define CKQ_ESCRATCH (-4) /* the call needs more scratch than the entry point that allocates nothing holds */
#define CKQ_ENOGROUP (-7) /* internal: a grouped GEMM launch was declined; the caller launches the matrices one by one */
#define CKQ_ENODUMP (-6)  /* the integer dumps are compiled into libckernel_quant_hip_dump.so only */
/* 1 in the test library (same sources, same templates, plus the DUMP instantiations that also
 * store the integers behind every output); 0 in the product library, which stays smaller for it. */
#ifndef CKQ_WITH_DUMP
#define CKQ_WITH_DUMP 0
#endif

/* Weight-format tags as in ckq_blocks.h, plus the fp32-activation variants
 * (X is then ntok rows of K floats). */
#define CKQ_KERNEL_Q80_F32 16
#define CKQ_KERNEL_Q4K_F32 17
#define CKQ_KERNEL_Q6K_F32 18

/*
 * y[t*ldy + row] = dot(W[row], X[t]) (+ bias[row]) for row < nrows, t < ntok.
 * W: nrows rows of K elements in `fmt` blocks; X: ntok activation rows
 * (Q8_K, or Q8_0 / fp32 for the Q8_0 weight kernels).
 * `row0`/`row1` restrict the computed rows to [row0,row1) (thread-split entry
 * points); outputs outside the range are not touched.
 * `subdots`, when non-NULL (at most eight tokens), runs the dump build of the
 * instantiation the call would otherwise run and receives the raw integer
 * sub-block dots, subdots[(t * nrows + row) * nsub + i]; y is not written.
 */
int ckq_launch_gemv(int fmt, float *y, const void *W, const void *X, const float *bias,
                    int nrows, int K, int ntok, long ldy, int row0, int row1,
                    int32_t *subdots, void *stream);

/* n (at most 4) independent matmuls of one format, input width and token count
 * (at most eight tokens; a token tile that does not fit in LDS is issued as
 * separate launches), problem i with rows[i] weight rows and output row stride
 * ldys[i], in one launch of the streaming kernel; the arrays are host arrays
 * (of device pointers), bias may be NULL or hold NULL entries.  `subdots`
 * non-NULL runs the dump build of the grouped kernel instead (y, ldys and bias
 * are then ignored): subdots[((g * ntok + t) * max_rows + row) * nsub + i]. */
int ckq_launch_gemv_group(int fmt, int n, float *const *y, const void *const *W, const void *const *X,
                          const float *const *bias, const int *rows, const long *ldys, int K, int ntok,
                          int32_t *subdots, void *stream);

/* n (2..4) weight matrices of one format against the same M x K quantized activations as one
 * matrix-core launch; CKQ_ENOGROUP when the matrices should be launched one by one instead. */
int ckq_launch_gemm_group(int fmt, int n, float *const *C, const void *const *B, const void *A,
                          const float *const *bias, const int *N, const long *ldc, int K, int M, void *stream);

/* The matrix-core GEMM of `fmt` for any token count, its integer block sums
 * stored next to the result: sums[((t * N + n) * nblk + b) * per + i]; nblk =
 * K / 256 and per = 2 (I1, I2) for Q4_K and Q5_K, per = 1 for Q6_K; nblk =
 * K / 32, per = 1 for Q8_0. */
int ckq_launch_gemm_block_sums(int fmt, const void *A, const void *B, const float *bias, float *C, int32_t *sums,
                               int M, int N, int K, long ldc, void *stream);

/* Kernel choice for more than eight tokens: 0 = by token count and weight size
 * (default), 1 = always the matrix-core GEMM, 2 = always the streaming kernel. */
void ckq_launch_set_gemm_policy(int policy);
/* Token tile of the Q4_K x Q8_K matrix-core GEMM: 0 = by shape (default), 64 or 96 = always that kernel. */
void ckq_launch_set_q4k_tile(int tokens);
/* Q6_K x Q8_K matrix-core GEMM: 0 = by shape (default), 1 = one block per CU always, 2 = the paired 64-token kernel always. */
void ckq_launch_set_q6k_variant(int variant);
/* Q5_K x Q8_K matrix-core GEMM: 0 = by tile count (default), 1 = one block per CU always, 2 = the paired kernel always. */
void ckq_launch_set_q5k_variant(int variant);

/* fp32 [rows x k] -> Q8_K / Q8_0 blocks, row-major. */
int ckq_launch_quantize_q8_k(const float *x, void *y, int rows, int k, void *stream);
int ckq_launch_quantize_q8_0(const float *x, void *y, int rows, int k, void *stream);

/* y[row] = Q8_K(SiLU(gate[row]) * up[row]), k floats per row, rows ld floats apart. */
int ckq_launch_swiglu_q8_k(const float *gate, const float *up, void *y, int rows, int k, long ld, void *stream);

/* RMSNorm over d_model floats per token (row stride aligned_embed_dim floats),
 * times gamma, quantized to Q8_K blocks: tokens x (d_model/256) blocks. */
int ckq_launch_rmsnorm_q8_k_fused(const float *input, const float *gamma, void *y, int tokens, int d_model,
                                  int aligned_embed_dim, float eps, void *stream);

/* Dequantize rows of a Q4_K / Q6_K / Q8_0 table to fp32: out[t] (n_row floats,
 * t < n_out_rows) = row (ids ? ids[t] clamped to [0,vocab) else t) for t <
 * tokens, plus pos[t] when pos is given, zero from element n_valid on; output
 * rows from `tokens` on are zero. */
int ckq_launch_dequant_rows(int fmt, const void *table, const int32_t *ids, int vocab, const float *pos,
                            float *out, int n_valid, int n_row, int tokens, int n_out_rows, void *stream);

/* ckq_launch_gemv for callers that must not allocate: a K-split matrix-core
 * GEMM takes its partial tiles from a static device array of
 * CKQ_NOALLOC_SCRATCH_BYTES instead of the grow-only workspace; a split that
 * needs more returns CKQ_ESCRATCH.  Formats Q4_K, Q5_K, Q6_K, Q8_0.
 * ckq_launch_noalloc_setup() resolves the array's address for the current
 * device (once per device; also done by the first call on a device). */
#define CKQ_NOALLOC_SCRATCH_BYTES ((size_t)4 << 20)
int ckq_launch_noalloc_setup(void);

/* Frees the K-split / rewrite scratch held for `stream` on the current device. */
int ckq_launch_release_stream(void *stream);

int ckq_launch_gemv_noalloc(int fmt, float *y, const void *W, const void *X, const float *bias,
                            int nrows, int K, int ntok, long ldy, void *stream);

/* Host arithmetic of launches chunked over gridDim.y (at most 65 535 token
 * tiles per launch): chunk c of `per` tokens out of `total` covers
 * [*first, *first + *count).  Exported for the index test. */
void ckq_grid_chunk(long total, long per, long c, long *first, long *count);

/* Plain device copy kernel (calibration of the memory counters / roofline). */
int ckq_launch_copy(void *dst, const void *src, size_t bytes, void *stream);
int ckq_launch_read(const void *src, size_t bytes, void *sink, void *stream);
int ckq_launch_read_tuned(const void *src, size_t bytes, void *sink, int blocks, int unroll, void *stream);

#ifdef __cplusplus
}
#endif
#endif
