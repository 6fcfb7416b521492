/*
 * ckq_producers.hpp - the activation producers (fp32 -> Q8_K, SiLU(gate)*up ->
 * Q8_K, RMSNorm -> Q8_K) as device functions: the arithmetic of the stand-alone
 * producer kernels of ckq_kernels.hip, kept apart from their launch shapes.
 */
#pragma once
#include "ckq_device.hpp"

/* ---- SiLU(gate) * up as the reference's tile loop evaluates it -------------
 * (fused/prefill_fused_gemm.c:904-906, 1034-1040): g / (1 + expf(-g)), then
 * the product, each operation rounded to fp32.  exp is evaluated in double
 * and rounded once, which agrees with a correctly rounded expf. */
__device__ __forceinline__ float swiglu_value(float g, float u)
{
#pragma clang fp contract(off)
    const float e = (float)exp(-(double)g);
    const float s = g / (1.0f + e);
    return s * u;
}

/* One wave: 256-block `blk` (of bpr per row, rows ldx floats apart) of x, or of
 * SiLU(x) * up, -> the Q8_K block at y + blk * 292. */
template <bool SWIGLU>
__device__ __forceinline__ void pro_quantize_block(const float *__restrict__ x, const float *__restrict__ up,
                                                   uint8_t *__restrict__ y, long blk, int bpr, long ldx, int lane)
{
    const long src = (blk / bpr) * ldx + (blk % bpr) * 256;
    const float4 v = reinterpret_cast<const float4 *>(x + src)[lane];
    float e[4] = {v.x, v.y, v.z, v.w};
    if constexpr (SWIGLU) {
        const float4 w = reinterpret_cast<const float4 *>(up + src)[lane];
        e[0] = swiglu_value(e[0], w.x); e[1] = swiglu_value(e[1], w.y);
        e[2] = swiglu_value(e[2], w.z); e[3] = swiglu_value(e[3], w.w);
    }
    q8k_quantize_block(e, lane, y + blk * 292);
}

/* ---- RMSNorm -> Q8_K (reference: src/kernels/fused/rmsnorm_q8_k_fused.c:54-142
 * as an FMA build compiles it) ------------------------------------------------
 * The sum of squares must be the reference's to the bit, or rstd moves by an
 * ulp and quants flip: eight strided lanes (lane j takes x[8i+j]) each a chain
 * of fused multiply-adds, combined as ((l0+l4)+(l1+l5)) + ((l2+l6)+(l3+l7)). */

/* Thread j < 8 of the block walks chain j over the row staged in LDS at xs
 * (D floats, D a multiple of 256) and leaves its sum at xs[D + j].  The chain
 * is serial; sixteen LDS reads are kept in flight ahead of it. */
__device__ __forceinline__ void rms_chain(float *xs, int D, int j)
{
    float acc = 0.0f, cur[16], nxt[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) cur[u] = xs[j + 8 * u];
    for (int d = 0; d < D; d += 128) {
        const int dn = d + 128 < D ? d + 128 : d;
#pragma unroll
        for (int u = 0; u < 16; ++u) nxt[u] = xs[dn + j + 8 * u];
#pragma unroll
        for (int u = 0; u < 16; ++u) acc = __fmaf_rn(cur[u], cur[u], acc);
#pragma unroll
        for (int u = 0; u < 16; ++u) cur[u] = nxt[u];
    }
    xs[D + j] = acc;
}

/* rstd from the eight chain sums (every thread derives the same value).
 * sqrtf and '/' are the correctly rounded ones (the __fsqrt_rn intrinsic is not). */
__device__ __forceinline__ float rms_rstd(const float *xs, int D, float eps)
{
    const float s04 = xs[D + 0] + xs[D + 4], s15 = xs[D + 1] + xs[D + 5];
    const float s26 = xs[D + 2] + xs[D + 6], s37 = xs[D + 3] + xs[D + 7];
    const float sum_sq = (s04 + s15) + (s26 + s37);
    return 1.0f / sqrtf(sum_sq / (float)D + eps);
}

/* One wave: n = (x*rstd)*gamma with two roundings, scale from the largest |n|
 * of the block (unlike quantize_row_q8_k's signed first-largest), iscale =
 * -127/max, d = 1/iscale, q = RNE(n*iscale) saturated; lane l owns 4l..4l+3. */
__device__ __forceinline__ void rms_quant_block(const float4 xv, const float4 gv, float rstd, int lane, uint8_t *out)
{
    const float e[4] = {__fmul_rn(__fmul_rn(xv.x, rstd), gv.x), __fmul_rn(__fmul_rn(xv.y, rstd), gv.y),
                        __fmul_rn(__fmul_rn(xv.z, rstd), gv.z), __fmul_rn(__fmul_rn(xv.w, rstd), gv.w)};
    float amax = fmaxf(fmaxf(fabsf(e[0]), fabsf(e[1])), fmaxf(fabsf(e[2]), fabsf(e[3])));
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    if (amax == 0.0f) {
        reinterpret_cast<u32 *>(out)[lane] = 0;
        if (lane < 9) reinterpret_cast<u32 *>(out)[64 + lane] = 0;
        return;
    }
    const float iscale = __fdiv_rn(-127.0f, amax);
    int q[4], sum = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        q[i] = rne_sat_i8(__fmul_rn(e[i], iscale));
        sum += q[i];
    }
    reinterpret_cast<u32 *>(out + 4)[lane] =
        (u32)(q[0] & 0xff) | ((u32)(q[1] & 0xff) << 8) | ((u32)(q[2] & 0xff) << 16) | ((u32)(q[3] & 0xff) << 24);
    sum = group_sum<4>(sum);
    if ((lane & 3) == 3) reinterpret_cast<int16_t *>(out + 260)[lane >> 2] = (int16_t)sum;
    if (lane == 0) *reinterpret_cast<float *>(out) = __fdiv_rn(1.0f, iscale);
}

/* One block of NW waves turns row x (D floats) into its D/256 Q8_K blocks at
 * y.  Wave w owns 256-blocks w, w + NW, ...; the gamma of its first GREG
 * blocks is loaded at the start and kept in registers across the chain, so a
 * single row costs one round trip to memory, not one per 256-block (x itself
 * comes back from LDS).  smem: D floats + 8. */
template <int NW, int GREG>
__device__ __forceinline__ void rms_row(const float *__restrict__ x, const float *__restrict__ gamma,
                                        uint8_t *__restrict__ y, int D, float eps, float *xs)
{
    const int tid = threadIdx.x, lane = tid & 63, wave = wave_in_block();
    const int nb = D / 256;
    float4 gv[GREG];
#pragma unroll
    for (int r = 0; r < GREG; ++r) {
        const int b = wave + NW * r;
        gv[r] = reinterpret_cast<const float4 *>(gamma + 256 * (b < nb ? b : nb - 1))[lane];
    }
    for (int b = wave; b < nb; b += NW)
        reinterpret_cast<float4 *>(xs + 256 * b)[lane] = reinterpret_cast<const float4 *>(x + 256 * b)[lane];
    __syncthreads();
    if (tid < 8) rms_chain(xs, D, tid);
    __syncthreads();
    const float rstd = rms_rstd(xs, D, eps);
#pragma unroll
    for (int r = 0; r < GREG; ++r) {
        const int b = wave + NW * r;
        if (b < nb) rms_quant_block(reinterpret_cast<const float4 *>(xs + 256 * b)[lane], gv[r], rstd, lane, y + (size_t)b * 292);
    }
    for (int b = wave + NW * GREG; b < nb; b += NW)
        rms_quant_block(reinterpret_cast<const float4 *>(xs + 256 * b)[lane],
                        reinterpret_cast<const float4 *>(gamma + 256 * b)[lane], rstd, lane, y + (size_t)b * 292);
}
