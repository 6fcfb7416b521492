/*
 * ckq_gemv.hpp - the weight-streaming dequant-dot kernel (decode GEMV and token
 * tiles of up to eight activation rows) and its launch-shape selection, as
 * templates over the per-format traits of ckq_formats.hpp.  Each format is
 * instantiated in a translation unit of its own (ckq_gemv_<fmt>.hip).
 */
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ckq_blocks.h"
#include "ckq_formats.hpp"
#include "ckq_launch.h"

constexpr int CKQ_GROUP_MAX = 4;   /* independent matmuls of one shape in one launch */

struct GemvArgs {
    float         *y;
    const uint8_t *W;
    const uint8_t *X;
    const float   *bias;
    int32_t       *sub;
    int  nrows, npos, ntok, row0, row1, nsub_row;
    long wrow, xrow, ldy;
};

/* Problems 1..3 of a grouped launch (blockIdx.z = g > 0); problem 0 is in GemvArgs. */
struct GemvGroup {
    float         *y[CKQ_GROUP_MAX - 1];
    const uint8_t *W[CKQ_GROUP_MAX - 1];
    const uint8_t *X[CKQ_GROUP_MAX - 1];
    const float   *bias[CKQ_GROUP_MAX - 1];
    int nrows[CKQ_GROUP_MAX - 1];           /* rows of each further problem (the grid covers the largest) */
    int ldy[CKQ_GROUP_MAX - 1];             /* and its output row stride */
    int n;                                  /* problems in the launch, 1 = not grouped */
};


/*
 * Tiled kernel (token tiles MT >= 1; DUMP: the same instantiation also stores
 * the raw integer sub-block dots of every (token, row), for the exactness tests).  One wave
 * handles (64/LPR)*RPI weight rows: LPR lanes share a row, lane l of the group
 * owns positions l, l+LPR, ... (PPL of them per pass).  All weight and
 * activation loads of a pass are issued before anything is decoded.  There is
 * no loop over rows: the grid supplies the parallelism.  The fp32 partials are
 * summed over the LPR lanes with a fixed DPP tree; the last lane of the group
 * stores.
 */
template <class F, int LPR, int PPL, int MT, int RPI, bool DUMP, int WPB, bool LDSX, bool GRP = false>
__global__ void __launch_bounds__(64 * WPB) __attribute__((amdgpu_waves_per_eu(DUMP ? 1 : MT == 1 && PPL == 1 && RPI == 1 ? F::OCC1 : MT == 1 && PPL == 1 && RPI == 2 && LPR == 64 ? F::OCC2 : MT >= 4 && PPL == 1 ? 4 : 1)))
gemv_kernel(const uint8_t *W, const uint8_t *X, long wrow, long xrow, int row0, int row1, int npos, int ntok,
            float *y, const float *bias, long ldy, int32_t *sub, int nsub_row, int nrows, GemvGroup grp)
{
    /* The arguments are scalars, those the first loads need in front: the
     * first fourteen registers' worth arrive preloaded with the wave (build
     * flag -amdgpu-kernarg-preload-count) instead of through a scalar load
     * that every wave waits for before it can issue its first weight load. */
    const int g = GRP ? (int)blockIdx.z : 0;
    const int row1g = GRP && g ? grp.nrows[g - 1] : row1;    /* problems of a group may differ in their row count */
    const long ldyg = GRP && g ? (long)grp.ldy[g - 1] : ldy;
    const GemvArgs a = {y, W, X, bias, sub, nrows, npos, ntok, row0, row1g, nsub_row, wrow, xrow, ldyg};
    constexpr int SLOTS = 64 / LPR;
    extern __shared__ __attribute__((aligned(16))) uint8_t xs[];   /* LDSX: the MT activation rows */
    /* grouped launch: blockIdx.z picks the problem (a separate instantiation: the extra
     * argument loads lengthen the start of every wave, which a bandwidth-bound launch
     * of a few microseconds feels) */
    float *const         gy    = g == 0 ? a.y    : grp.y[g - 1];
    const uint8_t *const gW    = g == 0 ? a.W    : grp.W[g - 1];
    const uint8_t *const gX    = g == 0 ? a.X    : grp.X[g - 1];
    const float *const   gbias = g == 0 ? a.bias : grp.bias[g - 1];
    const int lane = threadIdx.x & 63, wave = wave_in_block();
    const int slot = lane / LPR, l = lane % LPR;
    const int wave_row = a.row0 + (blockIdx.x * WPB + wave) * (SLOTS * RPI);   /* uniform */
    const bool live = wave_row < a.row1;
    if (!LDSX && !live) return;
    const int wrow_c = min(wave_row, a.row1 - 1);
    const int rbase = wave_row + slot * RPI;
    const int t0 = blockIdx.y * MT;
    /* dump layout: [problem of the group][token][row of nrows][sub-block] */
    const size_t dump_base = DUMP && GRP ? (size_t)g * a.ntok * a.nrows * a.nsub_row : 0;
    const uint8_t *wbase = gW + (size_t)wrow_c * a.wrow;                      /* uniform */

    /* Every wave of the block reads the same activation rows: they are staged
     * once in LDS instead of once per wave through the vector cache.  Their
     * loads go out first, all at once (one round trip, they hit in L2), the
     * weight loads follow, and only then are the staged values written. */
    constexpr int XNT = 64 * WPB, XU = MT == 1 ? 2 : 4;
    const int mt_live = min(MT, a.ntok - t0);
    const uint8_t *xsrc = gX + (size_t)t0 * (size_t)a.xrow;
    const int xbytes = (int)((long)mt_live * a.xrow), xn = xbytes / F::XS_SRC;   /* staging units */
    const u32 xcap = (u32)((long)MT * a.xrow / F::XS_SRC);                                     /* units of a full tile */
    u32 xv[XU][F::XS_REGS];
    if (LDSX) {
#pragma unroll
        for (int u = 0; u < XU; ++u) {
            const int i = u * XNT + (int)threadIdx.x;                 /* units past the tile re-read its last one */
            F::xs_ld(xv[u], xsrc + (u32)F::XS_SRC * (u32)min(i, xn - 1));
        }
    }

    float acc[RPI][MT];
#pragma unroll
    for (int r = 0; r < RPI; ++r)
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[r][t] = 0.0f;

    u32 rowoff[RPI];   /* byte offset of the lane's r-th row from wbase, clamped to the last row */
#pragma unroll
    for (int r = 0; r < RPI; ++r) rowoff[r] = (u32)(min(rbase + r, a.row1 - 1) - wrow_c) * (u32)a.wrow;

    for (int p0 = 0; p0 < a.npos; p0 += LPR * PPL) {
        typename F::Wt  w[RPI][PPL];
        typename F::Act act[MT >= 4 ? 1 : MT][PPL];   /* wide tiles stream their activations instead */
#pragma unroll
        for (int p = 0; p < PPL; ++p) {
            const int pos = min(p0 + p * LPR + l, a.npos - 1);
            const typename F::Off o = F::w_off(pos);
#pragma unroll
            for (int r = 0; r < RPI; ++r) {
                typename F::Off orow = o;
                F::off_shift(orow, rowoff[r]);
                F::load_w(w[r][p], wbase, orow);
            }
        }
        if (LDSX && p0 == 0) {
            /* the staged activations' loads are older than the weight loads
             * just issued, so waiting for them does not wait for the weights */
#pragma unroll
            for (int u = 0; u < XU; ++u) {
                const int i = u * XNT + (int)threadIdx.x;
                if (i < xn) F::xs_st(xs, xv[u], (u32)i, xcap);
            }
            for (int i = XNT * XU + (int)threadIdx.x; i < xn; i += XNT) {       /* long token tiles */
                u32 v[F::XS_REGS];
                F::xs_ld(v, xsrc + (u32)F::XS_SRC * (u32)i);
                F::xs_st(xs, v, (u32)i, xcap);
            }
            if (F::XS_SRC == 16) {
                const int tail = (xbytes & 15) >> 1;  /* plain-copy images: rows are a whole number of 2-byte units */
                if ((int)threadIdx.x < tail) {
                    const u32 o = 16u * (u32)xn + 2u * threadIdx.x;
                    *reinterpret_cast<uint16_t *>(xs + o) = (uint16_t)ld2(xsrc + o);
                }
            }
            __syncthreads();
        }
        if constexpr (MT >= 4) {
            /* wide token tiles: the weights of a position are decoded once, then
             * the tokens' activations stream through from LDS one at a time
             * (holding all of them in registers would leave two waves per SIMD) */
#pragma unroll
            for (int p = 0; p < PPL; ++p) {
                const int  upos  = p0 + p * LPR + l;
                const bool valid = upos < a.npos;
                const int  pos   = min(upos, a.npos - 1);
                typename F::Dec dec[RPI];
#pragma unroll
                for (int r = 0; r < RPI; ++r) F::decode(dec[r], w[r][p], pos);
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    typename F::Act at;
                    if (LDSX) {
                        const int tl = min(t, a.ntok - t0 - 1);                    /* uniform */
                        F::load_act_lds(at, xs, tl, pos, (u32)a.xrow, a.npos, xcap);
                    } else {
                        const int tok = min(t0 + t, a.ntok - 1);                   /* uniform */
                        F::load_act(at, gX + (size_t)tok * a.xrow, pos);
                    }
#pragma unroll
                    for (int r = 0; r < RPI; ++r) {
                        int sub[F::NSUB];
                        const float v = F::dot(dec[r], at, sub);
                        acc[r][t] += valid ? v : 0.0f;
                        if (DUMP && valid && rbase + r < a.row1 && t0 + t < a.ntok) {
#pragma unroll
                            for (int i = 0; i < F::NSUB; ++i)
                                a.sub[dump_base + ((size_t)(t0 + t) * a.nrows + (rbase + r)) * a.nsub_row + F::sub_index(pos, i)] = sub[i];
                        }
                    }
                }
            }
        } else {
#pragma unroll
        for (int p = 0; p < PPL; ++p) {
            const int pos = min(p0 + p * LPR + l, a.npos - 1);
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                if (LDSX) {
                    const int tl = min(t, a.ntok - t0 - 1);                    /* uniform */
                    F::load_act_lds(act[t][p], xs, tl, pos, (u32)a.xrow, a.npos, xcap);
                } else {
                    const int tok = min(t0 + t, a.ntok - 1);                   /* uniform */
                    F::load_act(act[t][p], gX + (size_t)tok * a.xrow, pos);
                }
            }
        }
#pragma unroll
        for (int p = 0; p < PPL; ++p) {
            const int  upos  = p0 + p * LPR + l;
            const bool valid = upos < a.npos;
            const int  pos   = min(upos, a.npos - 1);
#pragma unroll
            for (int r = 0; r < RPI; ++r) {
                typename F::Dec dec;
                F::decode(dec, w[r][p], pos);
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    int sub[F::NSUB];
                    const float v = F::dot(dec, act[t][p], sub);
                    acc[r][t] += valid ? v : 0.0f;
                    if (DUMP && valid && rbase + r < a.row1 && t0 + t < a.ntok) {
#pragma unroll
                        for (int i = 0; i < F::NSUB; ++i)
                            a.sub[dump_base + ((size_t)(t0 + t) * a.nrows + (rbase + r)) * a.nsub_row + F::sub_index(pos, i)] = sub[i];
                    }
                }
            }
        }
        }
    }

#pragma unroll
    for (int r = 0; r < RPI; ++r)
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const float s = group_sum<LPR>(acc[r][t]);
            const int row = rbase + r, tok = t0 + t;
            if (!DUMP && l == LPR - 1 && row < a.row1 && tok < a.ntok)
                gy[(size_t)tok * a.ldy + row] = gbias ? s + gbias[row] : s;
        }
}

/* Rows the grid has to cover: the computed range, or the largest problem of a group. */
static int launch_rows(const GemvArgs &a, const GemvGroup &grp) { return grp.n > 1 ? a.nrows : a.row1 - a.row0; }

/* Token tiles a launch can carry in gridDim.y; longer token lists go out as
 * several launches over consecutive token ranges (ckq_grid_chunk). */
constexpr int CKQ_GRID_Y_MAX = 65535;

template <class F, int LPR, int PPL, int MT, int RPI, bool DUMP, int WPB, bool LDSX>
static int launch_one(const GemvArgs &a0, const GemvGroup &grp, hipStream_t s)
{
    constexpr int rows_per_block = WPB * (64 / LPR) * RPI;
    const int nr = launch_rows(a0, grp);
    const size_t lds = LDSX ? F::xs_lds_bytes((size_t)MT * (size_t)a0.xrow) : 0;
    if (grp.n > 1) {
        if constexpr (LDSX) {                            /* grouped launches stage their activations in LDS */
            dim3 grid((nr + rows_per_block - 1) / rows_per_block, (a0.ntok + MT - 1) / MT, (unsigned)grp.n);
            hipLaunchKernelGGL((gemv_kernel<F, LPR, PPL, MT, RPI, DUMP, WPB, LDSX, true>), grid, dim3(64 * WPB), lds, s,
                               a0.W, a0.X, a0.wrow, a0.xrow, a0.row0, a0.row1, a0.npos, a0.ntok, a0.y, a0.bias, a0.ldy, a0.sub,
                               a0.nsub_row, a0.nrows, grp);
            return (int)hipGetLastError();
        }
        return CKQ_EINVAL;
    }
    const long per = (long)MT * CKQ_GRID_Y_MAX;
    if (a0.sub && a0.ntok > per) return CKQ_EINVAL;      /* the dump is indexed by the token of the whole call */
    for (long c = 0; c * per < a0.ntok; ++c) {
        long first, count;
        ckq_grid_chunk(a0.ntok, per, c, &first, &count);
        GemvArgs a = a0;
        a.X = a0.X + (size_t)first * (size_t)a0.xrow;
        a.y = a0.y ? a0.y + (size_t)first * (size_t)a0.ldy : nullptr;
        a.ntok = (int)count;
        dim3 grid((nr + rows_per_block - 1) / rows_per_block, (a.ntok + MT - 1) / MT, 1);
        hipLaunchKernelGGL((gemv_kernel<F, LPR, PPL, MT, RPI, DUMP, WPB, LDSX, false>), grid, dim3(64 * WPB), lds, s,
                           a.W, a.X, a.wrow, a.xrow, a.row0, a.row1, a.npos, a.ntok, a.y, a.bias, a.ldy, a.sub,
                           a.nsub_row, a.nrows, grp);
        const int rc = (int)hipGetLastError();
        if (rc) return rc;
    }
    return 0;
}

/* Activation rows are staged in LDS when the token tile fits in 64 KB.  The
 * dump build of an instantiation exists for the staged form only. */
template <class F, int LPR, int PPL, int MT, int RPI, int WPB>
static int launch_tile(const GemvArgs &a, const GemvGroup &grp, hipStream_t s)
{
    const bool fits = F::xs_lds_bytes((size_t)MT * (size_t)a.xrow) <= 65536;
    if (a.sub) {
#if CKQ_WITH_DUMP
        if constexpr (F::TOKEN_TILES) {
            if (fits) return launch_one<F, LPR, PPL, MT, RPI, true, WPB, true>(a, grp, s);
            if (MT == 1 && grp.n == 1) return launch_one<F, LPR, PPL, 1, 1, true, 4, false>(a, grp, s);
        }
        return CKQ_EINVAL;
#else
        return CKQ_ENODUMP;      /* the dump builds live in libckernel_quant_hip_dump.so */
#endif
    }
    if (fits) return launch_one<F, LPR, PPL, MT, RPI, false, WPB, true>(a, grp, s);
    return launch_one<F, LPR, PPL, MT, RPI, false, WPB, false>(a, grp, s);
}

/* Rows per wave-slot and waves per block for each token tile: one row per
 * slot in 256-thread blocks for the bandwidth-bound single-token case (as many
 * of the matrix's loads in flight as the CUs can hold, small barrier groups),
 * fewer rows in flight as the tile grows. */
template <class F, int LPR, int PPL>
static int launch_mt(const GemvArgs &a, const GemvGroup &grp, int max_mt, hipStream_t s)
{
    if (a.ntok == 1 || max_mt == 1) {
        /* 256-thread blocks; a second row per slot once the matrix needs more
         * than two rounds of resident waves anyway (halves the activation
         * staging per weight byte) */
        const long waves = ((long)launch_rows(a, grp) * LPR + 63) / 64;
        if (PPL == 1 && waves > 16384) return launch_tile<F, LPR, PPL, 1, 2, 4>(a, grp, s);
        /* rows longer than one pass: each staged activation row is shared
         * between eight weight rows, as 512-thread blocks (a whole number of
         * blocks per CU on the usual projection shapes) or, for the largest
         * matrices, two rows per slot */
        if (PPL > 1 && launch_rows(a, grp) >= 8192) return launch_tile<F, LPR, PPL, 1, 2, 4>(a, grp, s);
        if (PPL > 1 && launch_rows(a, grp) >= 2048) return launch_tile<F, LPR, PPL, 1, 1, 8>(a, grp, s);
        return launch_tile<F, LPR, PPL, 1, 1, 4>(a, grp, s);
    }
    if constexpr (F::TOKEN_TILES) {
        if (a.ntok == 2) return launch_tile<F, LPR, PPL, 2, 2, 4>(a, grp, s);
        if (a.ntok <= 4) return launch_tile<F, LPR, PPL, 4, 2, 4>(a, grp, s);
        return launch_tile<F, LPR, PPL, 8, 2, 4>(a, grp, s);   /* two rows per slot: the staged tile serves twice the weights */
    }
    return CKQ_EINVAL;   /* formats without token tiles are always launched with max_mt == 1 */
}

/* Entry of a format's translation unit: picks the lane mapping from the row
 * length.  a.sub non-NULL selects the dump build of the same instantiation. */
template <class F>
static int launch_fmt(const GemvArgs &a, const GemvGroup &grp, int max_mt, hipStream_t s)
{
    const int np = a.npos;
    if (np <= 8)  return launch_mt<F, 8, 1>(a, grp, max_mt, s);
    if (np <= 16) return launch_mt<F, 16, 1>(a, grp, max_mt, s);
    if (np <= 32) return launch_mt<F, 32, 1>(a, grp, max_mt, s);
    if (np <= 64) return launch_mt<F, 64, 1>(a, grp, max_mt, s);
    if (np <= 128) return launch_mt<F, 64, 2>(a, grp, max_mt, s);
    if (np <= 192) return launch_mt<F, 64, 3>(a, grp, max_mt, s);
    return launch_mt<F, 64, 4>(a, grp, max_mt, s);   /* longer rows loop in passes of 256 positions */
}

/* One function per trait, each defined in its own translation unit. */
int ckq_gemv_launch_q4k(const GemvArgs &a, const GemvGroup &grp, hipStream_t s);
int ckq_gemv_launch_q5k(const GemvArgs &a, const GemvGroup &grp, hipStream_t s);
int ckq_gemv_launch_q6k(const GemvArgs &a, const GemvGroup &grp, hipStream_t s);
int ckq_gemv_launch_q80(const GemvArgs &a, const GemvGroup &grp, hipStream_t s);
int ckq_gemv_launch_q80p(const GemvArgs &a, const GemvGroup &grp, hipStream_t s);
int ckq_gemv_launch_q50(const GemvArgs &a, const GemvGroup &grp, hipStream_t s);
int ckq_gemv_launch_q80_f32(const GemvArgs &a, const GemvGroup &grp, hipStream_t s);
int ckq_gemv_launch_q4k_f32(const GemvArgs &a, const GemvGroup &grp, hipStream_t s);
int ckq_gemv_launch_q6k_f32(const GemvArgs &a, const GemvGroup &grp, hipStream_t s);
