/*
 * ckq_blocks.h - GGUF-compatible quantization block layouts used by the
 * quantized dequant-dot kernels.
 *
 * These are the on-disk / in-memory formats the reference engine passes to
 * its kernels as `const void *W` / `const void *x_q8`:
 *   block_q8_0  reference include/ckernel_quant.h:104-107
 *   block_q4_K  reference include/ckernel_quant.h:124-129
 *   block_q6_K  reference include/ckernel_quant.h:139-144
 *   block_q8_K  reference include/ckernel_quant.h:153-157
 *   block_q5_K  reference src/kernels/gemm_kernels_q5_k.c:49-55 (file-local there)
 *
 * Names carry a ckq_ prefix so this header can be included next to the
 * reference's own header without clashing.
 */
#ifndef CKQ_BLOCKS_H
#define CKQ_BLOCKS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CKQ_QK_K   256 /* elements per K-quant super-block */
#define CKQ_QK8_0  32  /* elements per Q8_0 block */
#define CKQ_K_SCALE_SIZE 12

typedef uint16_t ckq_half; /* IEEE binary16 bit pattern */

/* Q8_0: 32 x int8 with one fp16 scale. 34 bytes, 2-byte aligned. */
typedef struct {
    ckq_half d;
    int8_t   qs[CKQ_QK8_0];
} ckq_block_q8_0;

/* Q5_0: 32 x 5-bit with one fp16 scale, value = d * (q - 16).  Element l < 16
 * is the low nibble of qs[l] with bit l of qh (little-endian 32-bit) as fifth
 * bit; element 16 + l the high nibble with bit 16 + l.  22 bytes, 2-byte
 * aligned (reference: include/ckernel_quant.h:60-75). */
typedef struct {
    ckq_half d;
    uint8_t  qh[4];
    uint8_t  qs[CKQ_QK8_0 / 2];
} ckq_block_q5_0;

/* Q4_K: 256 x 4-bit. fp16 d, fp16 dmin, 8 six-bit scales + 8 six-bit mins
 * packed in 12 bytes, 128 nibble bytes. 144 bytes (9 x 16 B).
 * For j in {0,64,128,192}: qs[j/2 + l] low nibble = element j+l,
 * high nibble = element j+32+l, l < 32. */
typedef struct {
    ckq_half d;
    ckq_half dmin;
    uint8_t  scales[CKQ_K_SCALE_SIZE];
    uint8_t  qs[CKQ_QK_K / 2];
} ckq_block_q4_K;

/* Q5_K: Q4_K plus a 32-byte plane of fifth bits. 176 bytes (11 x 16 B).
 * Bit 2g of qh[l] is the fifth bit of element 64g+l, bit 2g+1 of element
 * 64g+32+l. */
typedef struct {
    ckq_half d;
    ckq_half dmin;
    uint8_t  scales[CKQ_K_SCALE_SIZE];
    uint8_t  qh[CKQ_QK_K / 8];
    uint8_t  qs[CKQ_QK_K / 2];
} ckq_block_q5_K;

/* Q6_K: 256 x 6-bit (stored value - 32). 128 B low nibbles, 64 B high bit
 * pairs, 16 int8 sub-block scales, fp16 d LAST. 210 bytes, 2-byte aligned. */
typedef struct {
    uint8_t  ql[CKQ_QK_K / 2];
    uint8_t  qh[CKQ_QK_K / 4];
    int8_t   scales[CKQ_QK_K / 16];
    ckq_half d;
} ckq_block_q6_K;

/* Q8_K: activation super-block. fp32 d, 256 x int8, 16 x int16 sums of each
 * run of 16 quants. 292 bytes, 4-byte aligned. */
typedef struct {
    float    d;
    int8_t   qs[CKQ_QK_K];
    int16_t  bsums[CKQ_QK_K / 16];
} ckq_block_q8_K;

#define CKQ_BLOCK_Q8_0_SIZE 34
#define CKQ_BLOCK_Q5_0_SIZE 22
#define CKQ_BLOCK_Q4_K_SIZE 144
#define CKQ_BLOCK_Q5_K_SIZE 176
#define CKQ_BLOCK_Q6_K_SIZE 210
#define CKQ_BLOCK_Q8_K_SIZE 292

#if defined(__cplusplus)
#define CKQ_STATIC_ASSERT(c, m) static_assert(c, m)
#else
#define CKQ_STATIC_ASSERT(c, m) _Static_assert(c, m)
#endif
CKQ_STATIC_ASSERT(sizeof(ckq_block_q8_0) == CKQ_BLOCK_Q8_0_SIZE, "q8_0 size");
CKQ_STATIC_ASSERT(sizeof(ckq_block_q5_0) == CKQ_BLOCK_Q5_0_SIZE, "q5_0 size");
CKQ_STATIC_ASSERT(sizeof(ckq_block_q4_K) == CKQ_BLOCK_Q4_K_SIZE, "q4_K size");
CKQ_STATIC_ASSERT(sizeof(ckq_block_q5_K) == CKQ_BLOCK_Q5_K_SIZE, "q5_K size");
CKQ_STATIC_ASSERT(sizeof(ckq_block_q6_K) == CKQ_BLOCK_Q6_K_SIZE, "q6_K size");
CKQ_STATIC_ASSERT(sizeof(ckq_block_q8_K) == CKQ_BLOCK_Q8_K_SIZE, "q8_K size");
CKQ_STATIC_ASSERT(offsetof(ckq_block_q6_K, d) == 208, "q6_K d offset");
CKQ_STATIC_ASSERT(offsetof(ckq_block_q8_K, bsums) == 260, "q8_K bsums offset");
CKQ_STATIC_ASSERT(offsetof(ckq_block_q5_K, qs) == 48, "q5_K qs offset");

/* Weight / activation format tags used by the size helpers and the
 * synthetic-data generator. */
typedef enum {
    CKQ_FMT_Q4_K = 0,
    CKQ_FMT_Q5_K = 1,
    CKQ_FMT_Q6_K = 2,
    CKQ_FMT_Q8_0 = 3,
    CKQ_FMT_Q8_K = 4,
    CKQ_FMT_Q5_0 = 5
} ckq_format;

static inline int ckq_block_elems(int fmt)
{
    return (fmt == CKQ_FMT_Q8_0 || fmt == CKQ_FMT_Q5_0) ? CKQ_QK8_0 : CKQ_QK_K;
}

static inline size_t ckq_block_bytes(int fmt)
{
    switch (fmt) {
    case CKQ_FMT_Q4_K: return CKQ_BLOCK_Q4_K_SIZE;
    case CKQ_FMT_Q5_K: return CKQ_BLOCK_Q5_K_SIZE;
    case CKQ_FMT_Q6_K: return CKQ_BLOCK_Q6_K_SIZE;
    case CKQ_FMT_Q8_0: return CKQ_BLOCK_Q8_0_SIZE;
    case CKQ_FMT_Q8_K: return CKQ_BLOCK_Q8_K_SIZE;
    case CKQ_FMT_Q5_0: return CKQ_BLOCK_Q5_0_SIZE;
    default: return 0;
    }
}

/* Bytes of one row of k elements (k must be a multiple of the block size). */
static inline size_t ckq_row_bytes(int fmt, int k)
{
    return (size_t)(k / ckq_block_elems(fmt)) * ckq_block_bytes(fmt);
}

#ifdef __cplusplus
}
#endif
#endif /* CKQ_BLOCKS_H */
