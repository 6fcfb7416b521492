/*
 * ckq_gemm_mfma.cuh - prefill GEMM, Q4_K weights x Q8_K activations, on the
 * gfx950 int8 matrix cores.
 *
 *   C[t][n] = sum_b dx(t,b) * ( dw(n,b) * I1(t,n,b) - dmin(n,b) * I2(t,n,b) ) (+ bias[n])
 *   I1 = sum_j sc(n,b,j) * sum_{k in sub-block j} q4(n,k) * q8(t,k)      (exact int32)
 *   I2 = sum_j m(n,b,j)  * (bsums(t,b,2j) + bsums(t,b,2j+1))             (STORED bsums)
 * which is the arithmetic of the reference's token loop over
 * gemv_q4_k_q8_k (gemm_kernels_q4k_q8k.c:121-181, 283-326) with the integer
 * parts kept exact and one fp32 rounding sequence per 256-element block.
 *
 * Mapping to the hardware
 * - v_mfma_i32_32x32x32_i8: K = 32 is exactly one Q4_K sub-block.  A = 32
 *   tokens x 32 k (int8 activations), B = 32 k x 32 weight rows, D = 32x32
 *   int32.  Lane l supplies row/column l%32 and the 16 k of half l/32.
 * - The 6-bit sub-block scale cannot ride in an int8 operand (sc*q4 <= 945),
 *   and applying it to the int32 outputs costs one VALU op per output per
 *   sub-block, more than the MFMA itself.  Instead the weights are expanded to
 *   TWO int8 planes, H = (sc>>3)*q4 and L = (sc&7)*q4 (both <= 105), each
 *   accumulated over all eight sub-blocks of a block; I1 = 8*H + L exactly.
 *   Nibble unpack and the two multiplies (v_pk_mul_lo_u16 on byte pairs) are
 *   done once per weight and reused for every token sub-tile of the wave.
 * - The min term contracts 8 (min, bsum) pairs per block.  Stored bsums need
 *   13 bits; split as lo + 64*hi (lo in [0,63], hi in [-64,63]) both parts and
 *   the 6-bit mins are exact in bf16, so ONE v_mfma_f32_32x32x16_bf16 per
 *   32x32 tile per block yields I2 exactly in fp32 (|I2| < 2^24).
 * - Weights never touch LDS: each wave loads the 16-byte nibble runs of its 32
 *   rows straight into the lanes that need them as B operands (Q4_K stores
 *   sub-blocks 2g and 2g+1 as the low and high nibbles of the same bytes, so
 *   one 128-bit load feeds two K-steps).  Activations are staged per block
 *   through LDS with 272-byte rows so that ds_read_b128 of 32 token rows is
 *   bank-conflict free, double-buffered against the MFMA work.
 *
 * Block = 4 waves = (32*TS tokens) x (128 weight rows); wave w owns rows
 * 32w..32w+31.  Grid: token tiles fastest inside an XCD so the eight XCD L2s
 * each see a weight tile once.
 */
#pragma once
#include "ckq_device.cuh"

typedef int   ckq_v4i  __attribute__((ext_vector_type(4)));
typedef int   ckq_v16i __attribute__((ext_vector_type(16)));
typedef float ckq_v16f __attribute__((ext_vector_type(16)));
typedef __bf16 ckq_v8bf __attribute__((ext_vector_type(8)));
typedef unsigned short ckq_v2u16 __attribute__((ext_vector_type(2)));

struct GemmArgs {
    const uint8_t *A;     /* Q8_K activations, M rows of nb blocks */
    const uint8_t *B;     /* Q4_K weights, N rows of nb blocks */
    const float   *bias;  /* N or null */
    float         *C;     /* M x ldc */
    int  M, N, nb;
    long ldc;
    int  ntt, nnt;        /* token tiles, weight-row tiles */
};

#ifndef CKQ_GEMM_WPE
#define CKQ_GEMM_WPE 2          /* waves per SIMD the register budget is sized for */
#endif

constexpr int GEMM_XROW = 272;            /* padded LDS row: 256 quants + 16 */

/* packed u8x4 times a small scalar, byte-wise (every product < 256) */
__device__ __forceinline__ int mul_bytes(u32 v, u32 s16x2)
{
    const ckq_v2u16 a = __builtin_bit_cast(ckq_v2u16, v), b = __builtin_bit_cast(ckq_v2u16, s16x2);
    return __builtin_bit_cast(int, (ckq_v2u16)(a * b));
}

/* small non-negative / signed integer (|v| < 2^8 significant bits) -> bf16 bits */
__device__ __forceinline__ u32 bf16_bits(float f) { return __builtin_bit_cast(u32, f) >> 16; }

/* Staged activation block of BM tokens in LDS. */
template <int BM>
struct GemmTile {
    uint8_t  q[2][BM * GEMM_XROW];   /* int8 quants, 272-byte rows */
    float    d[2][BM];               /* block scale of each token */
    uint16_t b[2][BM * 16];          /* bf16: lo_0..7, 64*hi_0..7 of the stored bsums */
};

/* Weights of one 256-block for one lane: header + the 16-byte nibble runs of
 * its half of each 64-element group. */
struct GemmW {
    u32 hdr[4];
    u32 q[16];
};

__device__ __forceinline__ void gemm_load_w(GemmW &w, const uint8_t *wrow, int b, int half)
{
    const uint8_t *blk = wrow + (u32)b * 144u;
    ld16<4>(w.hdr, blk);
#pragma unroll
    for (int g = 0; g < 4; ++g) ld16<4>(w.q + 4 * g, blk + 16 + 32 * g + 16 * half);
}

/* One 256-block: expand the lane's weights to the two planes, run the MFMAs
 * against the staged activations of buffer `cur`, fold into the fp32 tile. */
template <int TS>
__device__ __forceinline__ void gemm_block(const GemmW &w, const GemmTile<32 * TS> &tile, int cur, int col, int half,
                                           ckq_v16f (&acc)[TS])
{
    /* 6-bit scales and mins of the 8 sub-blocks (word form of the unpack) */
    const u32 sc03 = w.hdr[1] & 0x3f3f3f3fu;
    const u32 sc47 = (w.hdr[3] & 0x0f0f0f0fu) | (((w.hdr[1] >> 6) & 0x03030303u) << 4);
    const u32 mn03 = w.hdr[2] & 0x3f3f3f3fu;
    const u32 mn47 = ((w.hdr[3] >> 4) & 0x0f0f0f0fu) | (((w.hdr[2] >> 6) & 0x03030303u) << 4);
    const float dw = h2f(w.hdr[0] & 0xffff), dmin = h2f(w.hdr[0] >> 16);

    ckq_v16i accH[TS], accL[TS];
#pragma unroll
    for (int ts = 0; ts < TS; ++ts)
#pragma unroll
        for (int r = 0; r < 16; ++r) { accH[ts][r] = 0; accL[ts][r] = 0; }

#pragma unroll
    for (int g = 0; g < 4; ++g) {
#pragma unroll
        for (int hi = 0; hi < 2; ++hi) {
            const int j = 2 * g + hi;
            const u32 scw = j < 4 ? sc03 : sc47;
            const u32 sc = (scw >> (8 * (j & 3))) & 0xff;
            const u32 mh = (sc >> 3) * 0x00010001u, ml = (sc & 7) * 0x00010001u;
            ckq_v4i bH, bL;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const u32 nib = hi ? ((w.q[4 * g + i] >> 4) & 0x0f0f0f0fu) : (w.q[4 * g + i] & 0x0f0f0f0fu);
                bH[i] = mul_bytes(nib, mh);
                bL[i] = mul_bytes(nib, ml);
            }
#pragma unroll
            for (int ts = 0; ts < TS; ++ts) {
                const ckq_v4i av = *reinterpret_cast<const ckq_v4i *>(
                    &tile.q[cur][(32 * ts + col) * GEMM_XROW + 32 * j + 16 * half]);
                accH[ts] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, bH, accH[ts], 0, 0, 0);
                accL[ts] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, bL, accL[ts], 0, 0, 0);
            }
        }
    }

    /* min term: B operand = the row's 8 mins as bf16, in both k halves */
    ckq_v8bf bm;
    {
        u32 m[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const u32 src = i < 2 ? mn03 : mn47;
            const u32 m0 = (src >> (16 * (i & 1))) & 0xff, m1 = (src >> (16 * (i & 1) + 8)) & 0xff;
            m[i] = bf16_bits((float)m0) | (bf16_bits((float)m1) << 16);
        }
        const ckq_v4i t = {(int)m[0], (int)m[1], (int)m[2], (int)m[3]};
        bm = __builtin_bit_cast(ckq_v8bf, t);
    }

#pragma unroll
    for (int ts = 0; ts < TS; ++ts) {
        const ckq_v4i ab = *reinterpret_cast<const ckq_v4i *>(&tile.b[cur][(32 * ts + col) * 16 + 8 * half]);
        ckq_v16f zero;
#pragma unroll
        for (int r = 0; r < 16; ++r) zero[r] = 0.0f;
        const ckq_v16f i2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(ckq_v8bf, ab), bm, zero, 0, 0, 0);
        /* fp32 combine; D layout: register r, lane l -> token row 8*(r/4) + 4*(l/32) + r%4 */
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            const float4 dx = *reinterpret_cast<const float4 *>(&tile.d[cur][32 * ts + 8 * r4 + 4 * half]);
            const float dxs[4] = {dx.x, dx.y, dx.z, dx.w};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int r = 4 * r4 + k;
                const float f = (float)((accH[ts][r] << 3) + accL[ts][r]);
                const float u = dw * f - dmin * i2[r];
                acc[ts][r] += u * dxs[k];
            }
        }
    }
}

template <int TS, int WPE>
__global__ void __launch_bounds__(256, WPE) gemm_q4k_mfma_kernel(GemmArgs a)
{
    constexpr int BM = 32 * TS;
    __shared__ __attribute__((aligned(16))) GemmTile<BM> tile;

    const int tid = threadIdx.x, lane = tid & 63, wave = wave_in_block();
    const int col = lane & 31, half = lane >> 5;

    /* block id -> (token tile, row tile); the token tiles of one row tile run
     * on the same XCD (blocks are dealt round-robin to the 8 XCDs) */
    const int id = blockIdx.x, xcd = id & 7, seq = id >> 3;
    const int tt = seq % a.ntt;
    const int nt = (seq / a.ntt) * 8 + xcd;
    if (nt >= a.nnt) return;
    const int t0 = tt * BM;
    const int n_lane = min(nt * 128 + wave * 32 + col, a.N - 1);            /* this lane's weight row */
    const uint8_t *wrow = a.B + (size_t)n_lane * a.nb * 144;
    const long xstride = (long)a.nb * 292;
    const int last = a.nb - 1;

    /* Staging roles.  Quants: 16 consecutive lanes cover the 256 contiguous
     * bytes of one token (coalesced), a wave covers 4 tokens per load, the
     * block 16; BM/16 loads per thread.  Side data (block scale and the 16
     * stored bsums): 4 lanes per token, 8 bytes of bsums each. */
    constexpr int NQ = BM / 16;
    const int sq_tok = tid >> 4, sq_c = tid & 15;
    const uint8_t *sq_src[NQ];
#pragma unroll
    for (int i = 0; i < NQ; ++i)
        sq_src[i] = a.A + (size_t)min(t0 + sq_tok + 16 * i, a.M - 1) * xstride + 4 + 16 * sq_c;
    const int st_tok = tid >> 2, st_q = tid & 3;                            /* BM <= 64 rows x 4 quarters */
    const bool st_live = st_tok < BM;
    const uint8_t *st_src = a.A + (size_t)min(t0 + st_tok, a.M - 1) * xstride;

    u32 nq[NQ][4];   /* a block's quant bytes staged by this thread */
    u32 nbs[2];      /* 4 stored bsums (sub-blocks 2q, 2q+1) of token st_tok */
    float nd = 0.f;
    auto stage_load = [&](int b) {
        const u32 boff = (u32)b * 292u;
#pragma unroll
        for (int i = 0; i < NQ; ++i) ld16<4>(nq[i], sq_src[i] + boff);
        ld8<4>(nbs, st_src + boff + 260 + 8 * st_q);
        nd = __builtin_bit_cast(float, ld4<4>(st_src + boff));
    };
    auto stage_store = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NQ; ++i)
            *reinterpret_cast<ckq_v4i *>(&tile.q[buf][(sq_tok + 16 * i) * GEMM_XROW + 16 * sq_c]) =
                ckq_v4i{(int)nq[i][0], (int)nq[i][1], (int)nq[i][2], (int)nq[i][3]};
        if (!st_live) return;
        if (st_q == 0) tile.d[buf][st_tok] = nd;
        /* sub-blocks j = 2q, 2q+1: B32 = bsums[2j] + bsums[2j+1] = lo + 64*hi */
        const int b0 = (int)(int16_t)(nbs[0] & 0xffff) + (int)(int16_t)(nbs[0] >> 16);
        const int b1 = (int)(int16_t)(nbs[1] & 0xffff) + (int)(int16_t)(nbs[1] >> 16);
        u32 *bd = reinterpret_cast<u32 *>(&tile.b[buf][st_tok * 16]);
        bd[st_q]     = bf16_bits((float)(b0 & 63)) | (bf16_bits((float)(b1 & 63)) << 16);
        bd[4 + st_q] = bf16_bits((float)(64 * (b0 >> 6))) | (bf16_bits((float)(64 * (b1 >> 6))) << 16);
    };

    ckq_v16f acc[TS];
#pragma unroll
    for (int ts = 0; ts < TS; ++ts)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[ts][r] = 0.0f;

    /* Two weight register sets alternate; every prefetch is unconditional
     * (block index clamped) so no set is ever a conditional copy. */
    GemmW w0, w1;
    stage_load(0);
    gemm_load_w(w0, wrow, 0, half);
    stage_store(0);
    __syncthreads();

    for (int b = 0; b < a.nb; b += 2) {
        /* issue the next block's global loads BEFORE the MFMA work of this
         * one; the scheduling barrier keeps the compiler from sinking them
         * down to their first use */
        stage_load(min(b + 1, last));
        gemm_load_w(w1, wrow, min(b + 1, last), half);
        __builtin_amdgcn_sched_barrier(0);
        gemm_block<TS>(w0, tile, 0, col, half, acc);
        __builtin_amdgcn_sched_barrier(0);
        stage_store(1);
        __syncthreads();

        stage_load(min(b + 2, last));
        gemm_load_w(w0, wrow, min(b + 2, last), half);
        __builtin_amdgcn_sched_barrier(0);
        if (b + 1 < a.nb) gemm_block<TS>(w1, tile, 1, col, half, acc);
        __builtin_amdgcn_sched_barrier(0);
        stage_store(0);
        __syncthreads();
    }

    /* store: lanes 0-31 / 32-63 write 32 consecutive floats of two token rows */
    const int n = nt * 128 + wave * 32 + col;
    if (n < a.N) {
        const float bias = a.bias ? a.bias[n] : 0.0f;
#pragma unroll
        for (int ts = 0; ts < TS; ++ts)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int t = t0 + 32 * ts + 8 * (r >> 2) + 4 * half + (r & 3);
                if (t < a.M) a.C[(size_t)t * a.ldc + n] = acc[ts][r] + bias;
            }
    }
}

static int launch_gemm_q4k_mfma(const void *A, const void *B, const float *bias, float *C,
                                int M, int N, int K, long ldc, hipStream_t s)
{
    GemmArgs g;
    g.A = (const uint8_t *)A; g.B = (const uint8_t *)B; g.bias = bias; g.C = C;
    g.M = M; g.N = N; g.nb = K / 256; g.ldc = ldc;
    constexpr int TS = 2;
    g.ntt = (M + 32 * TS - 1) / (32 * TS);
    g.nnt = (N + 127) / 128;
    const int nnt8 = (g.nnt + 7) / 8 * 8;
    hipLaunchKernelGGL((gemm_q4k_mfma_kernel<TS, CKQ_GEMM_WPE>), dim3(g.ntt * nnt8), dim3(256), 0, s, g);
    return (int)hipGetLastError();
}
