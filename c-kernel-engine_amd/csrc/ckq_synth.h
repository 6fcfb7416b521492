/*
 * ckq_synth.h - seeded synthetic data and GGUF-format weight encoders
 * (host-only helpers used to build benchmark and test inputs).
 */
#ifndef CKQ_SYNTH_H
#define CKQ_SYNTH_H

#include <stddef.h>
#include <stdint.h>
#include "../../include/ckq_blocks.h"

#ifdef __cplusplus
extern "C" {
#endif

/* fp32 streams: pure functions of (seed, index). */
void ckq_synth_normal(float *out, size_t n, float mean, float std, uint64_t seed);
void ckq_synth_uniform(float *out, size_t n, float lo, float hi, uint64_t seed);
void ckq_synth_bytes(uint8_t *out, size_t n, uint64_t seed);

uint16_t ckq_synth_fp32_to_fp16(float f);
float    ckq_synth_fp16_to_fp32(uint16_t h);

/* fp32 -> weight blocks, n elements (multiple of the block size). */
void ckq_synth_quantize_q4_k(const float *w, void *out, size_t n);
void ckq_synth_quantize_q5_k(const float *w, void *out, size_t n);
void ckq_synth_quantize_q6_k(const float *w, void *out, size_t n);
void ckq_synth_quantize_q8_0(const float *w, void *out, size_t n);
int  ckq_synth_quantize(int fmt, const float *w, void *out, size_t n);

/* [rows x k] matrix of N(mean,std) weights, quantized to fmt. */
int ckq_synth_weights(int fmt, void *out, int rows, int k, float mean, float std, uint64_t seed);

/* nblocks format-valid blocks with uniformly random payload bytes. */
int ckq_synth_random_blocks(int fmt, void *out, size_t nblocks, uint64_t seed);

#ifdef __cplusplus
}
#endif
#endif
