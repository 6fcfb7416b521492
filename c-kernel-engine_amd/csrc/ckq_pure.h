/*
 * ckq_pure.h - host-side helpers of the library that touch neither HIP nor
 * global state: index arithmetic, table bookkeeping, the manifest line
 * parser, the weight fingerprint.  Plain C, so that they can be built with
 * -fsanitize=address,undefined and driven by a CPU harness (oracle/asan_harness.c).
 */
#ifndef CKQ_PURE_H
#define CKQ_PURE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* FNV-1a over 64 samples of 64 bytes spread across [p, p + bytes), seeded with the size. */
uint64_t ckq_fingerprint(const void *p, size_t bytes);

/* Do [a, a + na) and [b, b + nb) intersect? */
int ckq_ranges_overlap(const void *a, size_t na, const void *b, size_t nb);

/* Row range [*r0, *r1) of thread ith of nth over M rows (reference:
 * gemm_kernels_q4k_q8k.c:226-231); `whole` != 0: ith 0 takes every row, the
 * others none.  Returns 0 when the thread has nothing to do. */
int ckq_split_rows(int M, int ith, int nth, int whole, int *r0, int *r1);

/* Token range [*first, *first + *count) of chunk c of a launch chunked over
 * gridDim.y in pieces of `per` tokens. */
void ckq_grid_chunk(long total, long per, long c, long *first, long *count);

/* Slot choice of the per-(device, stream, kind) scratch table: the slot whose
 * key equals `key`, else the first free one (key 0), else the least recently
 * used one (smallest last_use), which the caller recycles. */
int ckq_workspace_pick(const uint64_t *keys, const uint64_t *last_use, int n, uint64_t key);

/* One line of a weights manifest, name|dtype|file_offset|size|runtime_offset
 * (numbers in any C base).  The line is cut in place.  Returns 1 and fills
 * *size / *runtime_offset for a tensor of a quantized weight format the library
 * computes with (q4_k, q5_k, q6_k, q8_0, q5_0, with or without the underscore,
 * any case) and a non-zero size; 0 for comments, blank lines, other dtypes and
 * empty tensors; -1 for a line with fewer than five fields. */
int ckq_manifest_parse_line(char *line, unsigned long long *size, unsigned long long *runtime_offset);

#ifdef __cplusplus
}
#endif
#endif
