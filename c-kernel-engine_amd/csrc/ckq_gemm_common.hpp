/*
 * ckq_gemm_common.hpp - what the four matrix-core GEMM kernels share: operand
 * vector types, the launch arguments, the K-split bookkeeping and the entry
 * points of each kernel's translation unit.
 */
#pragma once
#include <mutex>
#include "ckq_device.hpp"
#include "ckq_launch.h"

typedef int   ckq_v4i  __attribute__((ext_vector_type(4)));
typedef int   ckq_v16i __attribute__((ext_vector_type(16)));
typedef float ckq_v16f __attribute__((ext_vector_type(16)));
typedef __bf16 ckq_v8bf __attribute__((ext_vector_type(8)));
typedef unsigned short ckq_v2u16 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) void ckq_lds_void;
typedef const __attribute__((address_space(1))) void ckq_glb_void;

/* One weight matrix of a grouped launch: several matrices that multiply the same activations (Q/K/V,
 * gate/up) share a grid; a matrix owns the block ids [id0, id0 + ntt * round_up(nnt, 8)). */
constexpr int GEMM_GROUP_MAX = 4;
struct GemmProblem {
    const uint8_t *B;
    const float   *bias;
    float         *C;
    long           ldc;
    int            N, nnt, id0;
};

struct GemmArgs {
    const uint8_t *A;     /* Q8_K activations, M rows of nb blocks */
    const uint8_t *B;     /* Q4_K weights, N rows of nb blocks */
    const float   *bias;  /* N or null */
    float         *C;     /* M x ldc */
    int  M, N, nb;
    long ldc;
    int  ntt, nnt;        /* token tiles, weight-row tiles */
    /* grouped launch: ngroup > 1 matrices, never split along K; B, bias, C, N, ldc, nnt above are those of grp[0] */
    int  ngroup;
    GemmProblem grp[GEMM_GROUP_MAX];
    /* split K: blockIdx.y = s handles K-steps [s * k_per, min(k_steps, (s + 1) * k_per)) and
     * writes its partial tile, without bias, to part + s * M * N (row pitch N) */
    int    splits, k_per;
    float *part;
    float *ext_part;       /* caller-provided scratch for `part` (launch options), or null */
    size_t ext_part_bytes;
    /* dump builds only: the exact integer block sums behind every output,
     * dump[((t * N + n) * nblk + b) * per + i] (per = 2: I1, I2 for Q4_K and
     * Q5_K; per = 1 for Q6_K and, with nblk = K / 32, for Q8_0) */
    int32_t *dump;
};

/* Where a lane of a dump build stores the sums of output (token offset `tok`
 * from the lane's first token, its row): nothing for rows or tokens outside
 * the matrix. */
/* A uniform value the compiler must take as new each time: keeps the 64 store
 * addresses of a dump from being hoisted out of the K loop into registers. */
__device__ __forceinline__ size_t gemm_opaque(size_t v)
{
    asm volatile("" : "+s"(v));
    return v;
}

struct GemmDumpLane {
    int32_t *p;          /* &dump[((t_first * N + n) * nblk + b) * per] */
    size_t   tok_stride; /* N * nblk * per */
    int      tok_left;   /* tokens from t_first to the end of the matrix */
    bool     row_ok;
    __device__ __forceinline__ void put(int tok, int i, int v) const
    {
        if (row_ok && tok < tok_left) p[(size_t)tok * tok_stride + i] = v;
    }
};

/* Launch options of the four GEMMs: `sums` non-NULL runs the dump build
 * (GemmArgs::dump); `scratch` non-NULL is caller-provided device memory of
 * scratch_bytes for the partial tiles of a K-split launch, used instead of the
 * library's grow-only workspace (nothing is allocated then; a split that needs
 * more returns CKQ_ESCRATCH). */
struct GemmOpts {
    int32_t *sums;
    float   *scratch;
    size_t   scratch_bytes;
};

/* What one block of a GEMM launch does: which tile id, which K-steps, where it
 * writes and whether it adds the bias. */
struct GemmOut { float *C; long ldc; const float *bias; };
struct GemmWork { int id, k0, k1; GemmOut out; const uint8_t *B; int N, nnt; };
__device__ __forceinline__ GemmWork gemm_work(const GemmArgs &a, int k_steps)
{
    const int id = blockIdx.x;
    if (a.ngroup > 1) {
        /* uniform selects, no indexing: the argument block stays in scalar registers */
        GemmProblem g = a.grp[0];
        if (id >= a.grp[1].id0) g = a.grp[1];
        if (a.ngroup > 2 && id >= a.grp[2].id0) g = a.grp[2];
        if (a.ngroup > 3 && id >= a.grp[3].id0) g = a.grp[3];
        return {id - g.id0, 0, k_steps, {g.C, g.ldc, g.bias}, g.B, g.N, g.nnt};
    }
    if (a.splits <= 1) return {id, 0, k_steps, {a.C, a.ldc, a.bias}, a.B, a.N, a.nnt};
    const int k0 = (int)blockIdx.y * a.k_per;
    return {id, k0, min(k_steps, k0 + a.k_per),
            {a.part + (size_t)blockIdx.y * (size_t)a.M * (size_t)a.N, (long)a.N, nullptr}, a.B, a.N, a.nnt};
}

/* Split K when the tile grid leaves most of the chip idle: `tiles` blocks of
 * `k_steps` loop iterations each.  Returns the number of splits (1 = none) so
 * that tiles * splits approaches the CU count while every split keeps at
 * least four iterations. */
static int gemm_choose_splits(int tiles, int k_steps)
{
    if (tiles >= 160 || k_steps < 8) return 1;
    int s = 256 / tiles;
    if (s > k_steps / 4) s = k_steps / 4;
    if (s > 16) s = 16;
    return s < 2 ? 1 : s;
}

constexpr int GEMM_TILE_ROWS = 128;    /* weight rows per tile, all four kernels */

/* Scratch for the partial tiles of K-split launches (kind 0) and for weights
 * rewritten for another kernel (kind 1): one grow-only device buffer per
 * stream and kind (work on one stream is ordered, so consecutive launches may
 * share it).  Growing it allocates and therefore synchronises.  The caller
 * holds gemm_split_mutex() from here until its last kernel is enqueued, so two
 * host threads launching on one stream cannot interleave their kernel pairs.
 * Defined in ckq_kernels.hip. */
std::recursive_mutex &gemm_split_mutex();
int gemm_workspace(int kind, hipStream_t s, size_t bytes, float **out);
/* C = bias + partial 0 + partial 1 + ... in that order (ckq_kernels.hip). */
int gemm_launch_reduce(float *C, long ldc, const float *part, const float *bias, int M, int N, int splits, hipStream_t s);

/* Common launch tail: sets up the split, launches `kernel` on grid (x, splits)
 * and, when split, the ordered reduction. */
template <class Kernel>
static int gemm_launch_split(Kernel kernel, GemmArgs &g, unsigned grid_x, int k_steps, hipStream_t s, unsigned threads = 256)
{
    g.splits = gemm_choose_splits(g.ntt * g.nnt, k_steps);
    g.k_per = (k_steps + g.splits - 1) / g.splits;
    g.splits = (k_steps + g.k_per - 1) / g.k_per;          /* no empty split */
    g.part = nullptr;
    if (g.splits <= 1) {
        hipLaunchKernelGGL(kernel, dim3(grid_x, 1u), dim3(threads), 0, s, g);
        return (int)hipGetLastError();
    }
    const size_t need = (size_t)g.splits * (size_t)g.M * (size_t)g.N * sizeof(float);
    if (g.ext_part) {
        /* caller-provided scratch: nothing is allocated and nothing is locked
         * (calls that share the scratch must not overlap).  Every partial
         * entry the reduction reads is written by the split kernel first, so
         * the scratch needs no clearing. */
        if (need > g.ext_part_bytes) return CKQ_ESCRATCH;
        g.part = g.ext_part;
        hipLaunchKernelGGL(kernel, dim3(grid_x, (unsigned)g.splits), dim3(threads), 0, s, g);
        const int rc = (int)hipGetLastError();
        if (rc) return rc;
        return gemm_launch_reduce(g.C, g.ldc, g.part, g.bias, g.M, g.N, g.splits, s);
    }
    std::lock_guard<std::recursive_mutex> lock(gemm_split_mutex());
    int rc = gemm_workspace(0, s, need, &g.part);
    if (rc) return rc;
    hipLaunchKernelGGL(kernel, dim3(grid_x, (unsigned)g.splits), dim3(threads), 0, s, g);
    rc = (int)hipGetLastError();
    if (rc) return rc;
    return gemm_launch_reduce(g.C, g.ldc, g.part, g.bias, g.M, g.N, g.splits, s);
}


/* packed u16x2 multiply-add, lane-wise (v_pk_mad_u16) */
__device__ __forceinline__ u32 pk_mad_u16(u32 a, u32 b, u32 c)
{
    const ckq_v2u16 x = __builtin_bit_cast(ckq_v2u16, a), y = __builtin_bit_cast(ckq_v2u16, b),
                    z = __builtin_bit_cast(ckq_v2u16, c);
    return __builtin_bit_cast(u32, (ckq_v2u16)(x * y + z));
}

/* acc += u * (lane 16*(l/16) + R of x): the multiply-add takes its first factor
 * from lane R of the caller's 16-lane row (DPP row_newbcast), so sixteen values
 * held one per lane serve sixteen instructions without being spread out first.
 * x must come from memory (LDS), not from a VALU instruction right before. */
__device__ __forceinline__ float fmac_row_lane(float acc, float x, float u, int r)
{
#define CKQ_BC(R) case R: asm("v_fmac_f32_dpp %0, %1, %2 row_newbcast:" #R " row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(x), "v"(u)); break;
    switch (r) {
        CKQ_BC(0) CKQ_BC(1) CKQ_BC(2) CKQ_BC(3) CKQ_BC(4) CKQ_BC(5) CKQ_BC(6) CKQ_BC(7)
        CKQ_BC(8) CKQ_BC(9) CKQ_BC(10) CKQ_BC(11) CKQ_BC(12) CKQ_BC(13) CKQ_BC(14) CKQ_BC(15)
    }
#undef CKQ_BC
    return acc;
}

/* A value that a VALU instruction computed, made safe as the x of fmac_row_lane: a DPP
 * instruction must not read a register a VALU instruction wrote in the two issue slots before it. */
__device__ __forceinline__ float dpp_source(float x)
{
    asm volatile("s_nop 1" : "+v"(x));
    return x;
}

/* Which token of its 32-token group output r = (lane & 15) of a lane is (the 32x32 MFMA result layout:
 * register r of lane l is row 8 (r / 4) + 4 (l / 32) + r % 4, column l % 32). */
__device__ __forceinline__ int mfma32_row_of_lane(int lane)
{
    return 8 * ((lane & 15) >> 2) + 4 * (lane >> 5) + (lane & 3);
}

/* A result leaves the chip once: the K-quant kernels store theirs non-temporally (whole 128-byte runs per wave
 * instruction; a tile's results are not read again by the launch that writes them, and the next launch runs on other
 * XCDs' L2s anyway): 1-2 % per launch.  The Q8_0 kernel, whose lanes store 16 bytes each to different rows, is 5-14 %
 * slower that way and keeps plain stores. */
#ifndef CKQ_GEMM_NT_STORE
#define CKQ_GEMM_NT_STORE 1
#endif
__device__ __forceinline__ void gemm_store(float *p, float v)
{
#if CKQ_GEMM_NT_STORE
    __builtin_nontemporal_store(v, p);
#else
    *p = v;
#endif
}

/* Grouped launch: the matrices of `in` against the same M x K activations, as one grid (no K split; the
 * callers group only what fills the chip without one).  rows_per_tile = weight rows of a block's tile. */
struct GemmGroupIn {
    int          n;
    const void  *B[GEMM_GROUP_MAX];
    const float *bias[GEMM_GROUP_MAX];
    float       *C[GEMM_GROUP_MAX];
    int          N[GEMM_GROUP_MAX];
    long         ldc[GEMM_GROUP_MAX];
};
/* Below this many tiles a single matrix is split along K instead (gemm_choose_splits); a group is not. */
constexpr int GEMM_GROUP_MIN_TILES = 160;
static int gemm_group_tiles(const GemmGroupIn &in, int M, int tokens_per_tile, int rows_per_tile = GEMM_TILE_ROWS)
{
    int tiles = 0;
    for (int p = 0; p < in.n; ++p)
        tiles += ((M + tokens_per_tile - 1) / tokens_per_tile) * ((in.N[p] + rows_per_tile - 1) / rows_per_tile);
    return tiles;
}
template <class Kernel>
static int gemm_launch_grouped(Kernel kernel, GemmArgs &g, const GemmGroupIn &in, hipStream_t s, unsigned threads = 256)
{
    unsigned grid = 0;
    g.ngroup = in.n;
    for (int p = 0; p < in.n; ++p) {
        const int nnt = (in.N[p] + GEMM_TILE_ROWS - 1) / GEMM_TILE_ROWS;
        g.grp[p] = {(const uint8_t *)in.B[p], in.bias[p], in.C[p], in.ldc[p], in.N[p], nnt, (int)grid};
        grid += (unsigned)g.ntt * (unsigned)((nnt + 7) / 8 * 8);
    }
    g.B = g.grp[0].B; g.bias = g.grp[0].bias; g.C = g.grp[0].C; g.N = g.grp[0].N; g.ldc = g.grp[0].ldc; g.nnt = g.grp[0].nnt;
    g.splits = 1; g.k_per = 0; g.part = nullptr;
    hipLaunchKernelGGL(kernel, dim3(grid, 1u), dim3(threads), 0, s, g);
    return (int)hipGetLastError();
}

/* The four kernels, one translation unit each: C[m*ldc + n] = dot(B row n, A row m) (+ bias[n]).
 * See GemmOpts for the options.  The _group forms return CKQ_ENOGROUP when the matrices are better
 * launched one by one (too few tiles to fill the chip without a K split). */
int launch_gemm_q4k_mfma_group(const void *A, const GemmGroupIn &in, int M, int K, hipStream_t s);
int launch_gemm_q5k_mfma_group(const void *A, const GemmGroupIn &in, int M, int K, hipStream_t s);
int launch_gemm_q6k_mfma_group(const void *A, const GemmGroupIn &in, int M, int K, hipStream_t s);
int launch_gemm_q80_mfma_group(const void *A, const GemmGroupIn &in, int M, int K, hipStream_t s);
int launch_gemm_q4k_mfma(const void *A, const void *B, const float *bias, float *C, int M, int N, int K, long ldc, const GemmOpts &opts, hipStream_t s);
int launch_gemm_q5k_mfma(const void *A, const void *B, const float *bias, float *C, int M, int N, int K, long ldc, const GemmOpts &opts, hipStream_t s);
int launch_gemm_q6k_mfma(const void *A, const void *B, const float *bias, float *C, int M, int N, int K, long ldc, const GemmOpts &opts, hipStream_t s);
int launch_gemm_q80_mfma(const void *A, const void *B, const float *bias, float *C, int M, int N, int K, long ldc, const GemmOpts &opts, hipStream_t s);
