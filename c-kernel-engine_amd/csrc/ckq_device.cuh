/*
 * ckq_device.cuh - gfx950 device helpers shared by the quantized kernels:
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
