/*
 * ckq_device.hpp - gfx950 device helpers shared by the quantized kernels:
 * unaligned 128-bit loads, packed int8 dot, wave64 DPP reductions.
 */
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint32_t u32;

/* GGUF blocks are only 2- or 4-byte aligned (Q6_K 210 B, Q8_0 34 B, Q8_K
 * 292 B).  Global loads on gfx950 run in unaligned-access mode, so a packed
 * struct with the true alignment still compiles to one global_load_dwordx4. */
template <int ALIGN> struct __attribute__((packed, aligned(ALIGN))) ckq_v4 { u32 v[4]; };
template <int ALIGN> struct __attribute__((packed, aligned(ALIGN))) ckq_v2 { u32 v[2]; };
template <int ALIGN> struct __attribute__((packed, aligned(ALIGN))) ckq_v1 { u32 v; };

template <int ALIGN, typename T>
__device__ __forceinline__ void ld16(T *dst, const uint8_t *p)
{
    const ckq_v4<ALIGN> t = *reinterpret_cast<const ckq_v4<ALIGN> *>(p);
    dst[0] = (T)t.v[0]; dst[1] = (T)t.v[1]; dst[2] = (T)t.v[2]; dst[3] = (T)t.v[3];
}
template <int ALIGN, typename T>
__device__ __forceinline__ void ld8(T *dst, const uint8_t *p)
{
    const ckq_v2<ALIGN> t = *reinterpret_cast<const ckq_v2<ALIGN> *>(p);
    dst[0] = (T)t.v[0]; dst[1] = (T)t.v[1];
}
template <int ALIGN>
__device__ __forceinline__ u32 ld4(const uint8_t *p)
{
    return reinterpret_cast<const ckq_v1<ALIGN> *>(p)->v;
}
__device__ __forceinline__ u32 ld2(const uint8_t *p)
{
    return *reinterpret_cast<const uint16_t *>(p);
}

/* Four signed int8 products accumulated into int32 (v_dot4_i32_i8). */
__device__ __forceinline__ int dot4(int a, int b, int c) { return __builtin_amdgcn_sdot4(a, b, c, false); }

__device__ __forceinline__ int mul24(int a, int b) { return __mul24(a, b); }

/* IEEE binary16 bit pattern -> fp32 (v_cvt_f32_f16; subnormals preserved). */
__device__ __forceinline__ float h2f(u32 h)
{
    return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

/* Sign-extend byte `idx` (0..3) of a dword. */
__device__ __forceinline__ int sbyte(u32 v, int idx) { return (int)(v << (24 - 8 * idx)) >> 24; }

/* Wave index as a scalar: lets the compiler keep row indices, row base
 * addresses and loop control in SGPRs (uniform branches, scalar address math). */
__device__ __forceinline__ int wave_in_block() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)); }

/* ---- DPP reductions -------------------------------------------------------
 * Fixed summation tree, so results do not depend on scheduling. */
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ float dpp_get(float v)
{
    return __builtin_bit_cast(float,
        __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, true));
}
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ int dpp_get(int v)
{
    return __builtin_amdgcn_update_dpp(0, v, CTRL, ROW_MASK, 0xF, true);
}

/* Sum over groups of LANES consecutive lanes (LANES in 4,8,16,32,64).  The
 * group total ends up in the LAST lane of every group (for 4/8/16 in every
 * lane of the group). */
template <int LANES, typename T>
__device__ __forceinline__ T group_sum(T v)
{
    v += dpp_get<0xB1>(v);                    /* quad_perm [1,0,3,2] */
    v += dpp_get<0x4E>(v);                    /* quad_perm [2,3,0,1] */
    if (LANES >= 8) v += dpp_get<0x141>(v);   /* row_half_mirror */
    if (LANES >= 16) v += dpp_get<0x140>(v);  /* row_mirror */
    if (LANES >= 32) v += dpp_get<0x142, 0xA>(v); /* row_bcast15 into rows 1,3 */
    if (LANES >= 64) v += dpp_get<0x143, 0xC>(v); /* row_bcast31 into rows 2,3 */
    return v;
}

/* x86 cvtps2dq + saturating packs (quantize_row_q8_k_sse.c:61-68): round to
 * nearest even; NaN, +-inf and anything outside int32 convert to INT_MIN, which
 * the packs saturate to -128 - also for +inf and for values >= 2^31 (a block of
 * magnitudes below 127/FLT_MAX has an infinite inverse scale). */
__device__ __forceinline__ int rne_sat_i8(float p)
{
    if (!(p < 2147483648.0f)) return -128;     /* NaN, +inf, >= 2^31 */
    const float r = __builtin_rintf(p);
    return (int)fminf(fmaxf(r, -128.0f), 127.0f);
}

/* One wave turns 256 fp32 values (lane l holds elements 4l..4l+3 in e) into
 * the 292-byte Q8_K block at `out` (global or LDS), with the reference's rules
 * (quantize_row_q8_k_sse.c:22-82): the scale comes from the FIRST element of
 * largest magnitude, sign kept, iscale = -127/max, q = RNE(x*iscale)
 * saturated, bsums over 16 elements, d = 1/iscale; an all-zero block is 292
 * zero bytes. */
__device__ __forceinline__ void q8k_quantize_block(const float (&e)[4], int lane, uint8_t *out)
{
    float amax = 0.0f, smax = 0.0f;
    int idx = 4 * lane;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float ax = fabsf(e[i]);
        if (ax > amax) { amax = ax; smax = e[i]; idx = 4 * lane + i; }
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float oa = __shfl_xor(amax, off), os = __shfl_xor(smax, off);
        const int   oi = __shfl_xor(idx, off);
        if (oa > amax || (oa == amax && oi < idx)) { amax = oa; smax = os; idx = oi; }
    }
    if (amax == 0.0f) {
        reinterpret_cast<u32 *>(out)[lane] = 0;
        if (lane < 9) reinterpret_cast<u32 *>(out)[64 + lane] = 0;
        return;
    }
    const float iscale = -127.0f / smax;
    int q[4], s = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        q[i] = rne_sat_i8(__fmul_rn(e[i], iscale));
        s += q[i];
    }
    const u32 packed = (u32)(q[0] & 0xff) | ((u32)(q[1] & 0xff) << 8) | ((u32)(q[2] & 0xff) << 16) | ((u32)(q[3] & 0xff) << 24);
    reinterpret_cast<u32 *>(out + 4)[lane] = packed;
    s = group_sum<4>(s);                       /* 16 consecutive elements = 4 lanes */
    if ((lane & 3) == 3) reinterpret_cast<int16_t *>(out + 260)[lane >> 2] = (int16_t)s;
    if (lane == 0) *reinterpret_cast<float *>(out) = 1.0f / iscale;
}
