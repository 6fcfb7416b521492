/*
 * ckq_gemm_q4k.hpp - what the Q4_K x Q8_K matrix-core kernels (ckq_gemm_q4k.hip: 64-token tiles,
 * ckq_gemm_q4k_t96.hip: 96-token tiles) share.
 */
#pragma once
#include "ckq_gemm_common.hpp"

#ifndef CKQ_GEMM_WPE
#define CKQ_GEMM_WPE 2          /* waves per SIMD the register budget is sized for */
#endif

/* packed u8x4 times a small scalar, byte-wise (every product < 256) */
__device__ __forceinline__ int mul_bytes(u32 v, u32 s16x2)
{
    const ckq_v2u16 a = __builtin_bit_cast(ckq_v2u16, v), b = __builtin_bit_cast(ckq_v2u16, s16x2);
    return __builtin_bit_cast(int, (ckq_v2u16)(a * b));
}

/* two floats whose low 16 bits are zero (integers of at most 8 significant
 * bits) -> their bf16 forms in one dword, lo in the low half: one v_perm_b32 */
__device__ __forceinline__ u32 bf16_pair(float lo, float hi)
{
    return __builtin_amdgcn_perm(__builtin_bit_cast(u32, hi), __builtin_bit_cast(u32, lo), 0x07060302u);
}

/* 96-token tiles, one block per tile, no K split (ckq_gemm_q4k_t96.hip).  g: A, B, bias, C, M, N, nb, ldc, nnt
 * and the dump pointer set by the caller; for the grouped form A, M and nb. */
int gemm_q4k_t96_token_tiles(int M);
int launch_gemm_q4k_t96(GemmArgs g, hipStream_t s);
int launch_gemm_q4k_t96_group(GemmArgs g, const GemmGroupIn &in, hipStream_t s);
