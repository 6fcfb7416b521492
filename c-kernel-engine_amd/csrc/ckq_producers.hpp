/*
 * ckq_producers.hpp - the activation producers (fp32 -> Q8_K, SiLU(gate)*up ->
 * Q8_K, RMSNorm -> Q8_K) as device functions, shared by their stand-alone
 * kernels and by the producer blocks at the front of a fused matmul launch, so
 * that both write the same bits; and the completion counter through which the
 * matmul blocks of such a launch learn that their activations exist.
 *
 * A fused launch (gemv_pro_kernel): the first `nblocks` blocks of grid x run
 * the producer, every other block is a matmul block that waits, resident and
 * with nothing in flight, until the producers have counted up to `target`,
 * and then runs as it would in a launch of its own.  What the fusion saves is
 * the boundary between two dependent launches (the producer's end-of-kernel
 * cache write-back, the next dispatch, its ramp): the matmul's waves are
 * already on the chip when the activations appear.  Block 0 is dispatched
 * first and never waits for anything, so the wait always ends; it is bounded
 * all the same (spin_limit polls), and an expired wait is recorded in flag[1].
 */
#pragma once
#include "ckq_device.hpp"

enum { CKQ_PRO_QUANT_Q8K = 1, CKQ_PRO_RMSNORM_Q8K = 2, CKQ_PRO_SWIGLU_Q8K = 3 };

struct GemvPro {
    const float *src;      /* fp32 rows (the gate rows of SwiGLU) */
    const float *src2;     /* gamma (RMSNorm) / up rows (SwiGLU) / unused */
    uint8_t     *dst;      /* rows x (k/256) Q8_K blocks */
    unsigned    *flag;     /* flag[0]: producer blocks completed since the counter was created; flag[1]: expired waits */
    unsigned     target;   /* flag[0] once every producer block of this launch has finished */
    int          spin_limit;
    int          nap;      /* naps of ~0.25 us between two polls of a waiting block */
    int          kind, nblocks, rows, k;
    long         ld;       /* floats between rows of src (and src2 for SwiGLU) */
    float        eps;
};

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

/* ---- producer blocks and the completion counter of a fused launch --------- */

/* Producer block `pb` of a fused launch (a block of WPB waves). */
template <int WPB>
__device__ __forceinline__ void pro_block(const GemvPro &pro, int pb, uint8_t *smem)
{
    const int lane = threadIdx.x & 63, wave = wave_in_block();
    const int bpr = pro.k / 256;
    if (pro.kind == CKQ_PRO_RMSNORM_Q8K) {
        if (pb < pro.rows)
            rms_row<WPB, 8 / WPB>(pro.src + (size_t)pb * pro.ld, pro.src2, pro.dst + (size_t)pb * bpr * 292, pro.k, pro.eps,
                                   reinterpret_cast<float *>(smem));
    } else {
        const long blk = (long)pb * WPB + wave, total = (long)pro.rows * bpr;
        if (blk < total) {
            if (pro.kind == CKQ_PRO_SWIGLU_Q8K) pro_quantize_block<true>(pro.src, pro.src2, pro.dst, blk, bpr, pro.ld, lane);
            else pro_quantize_block<false>(pro.src, nullptr, pro.dst, blk, bpr, pro.ld, lane);
        }
    }
    /* every wave makes its stores visible to the device, then one thread counts the block */
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    __syncthreads();
    if (threadIdx.x == 0) __hip_atomic_fetch_add(pro.flag, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}

/* Number of producer blocks of WPB waves each. */
static inline int pro_block_count(int kind, int rows, int k, int wpb)
{
    if (kind == CKQ_PRO_RMSNORM_Q8K) return rows;
    const long total = (long)rows * (k / 256);
    return (int)((total + wpb - 1) / wpb);
}

/* A matmul block of a fused launch: wait (bounded) until the producers of this
 * launch have all counted.  The activations are read only after this, with
 * ordinary loads and WITHOUT a cache invalidate: the producers have written
 * them back to memory (their release), and no cache on the reader's side can
 * hold an older copy of those lines - the launch began with the queue's
 * acquire, no matmul block touches the activations before its wait has ended,
 * and the host refuses to fuse when their cache lines are shared with anything
 * the matmul blocks read earlier (the weights).  An invalidate per block would
 * be correct too, but one per block of a launch of thousands costs ten times
 * the launch (measured: 36-91 us against 8-12). */
__device__ __forceinline__ void pro_wait(const GemvPro &pro)
{
    if (threadIdx.x == 0) {
        int n = 0;
        while ((int)(__hip_atomic_load(pro.flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - pro.target) < 0) {
            if (++n > pro.spin_limit) {
                __hip_atomic_fetch_add(pro.flag + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                break;
            }
            for (int k = 0; k < pro.nap; ++k) __builtin_amdgcn_s_sleep(8);     /* ~0.25 us per nap */
        }
    }
    __syncthreads();
}
